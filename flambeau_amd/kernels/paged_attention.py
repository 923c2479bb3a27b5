"""The kernel set of grouped-query attention over a paged cache: the joined q/k/v projection with
rotation and stores, attention itself, and what the kernels want prepared per step.

``PlainPagedAttention`` is the 32-bit path (and bfloat16 with the tuned kernels switched off): one
kernel per operation, nothing to prepare.  ``TunedPagedAttention`` sends rows of short portions to the
split-K kernel and longer portions to the tiled one (``kernels/tuned.py`` holds their shape rules)."""
from __future__ import annotations

from . import ops
from .sets import register_kernel_set


class PlainPagedAttention:
    def __init__(self, rt):
        self.rt = rt

    def row_order(self, n_heads: int, n_kv_heads: int, head_dim: int, rotated_dims: int):
        """The order in which the rows of a joined q/k/v matrix have to lie for ``project_rotate_store``
        (a permutation), or ``None`` where the kernels read them as they are."""
        return None

    def project_rotate_store(self, x, w, step, table, angles, q_out, kv, n_heads: int, rotated_dims: int, writes: bool) -> bool:
        """The joined q/k/v projection fused with rotation and the stores of q (into ``q_out``) and of
        the cache rows (into ``kv`` where ``writes``); the rows of ``w`` lie in ``row_order``, ``angles``
        are the step's cosines and sines.  ``False`` if no kernel takes the shape: the caller then runs
        product and rotation apart."""
        return False

    def attention(self, q, out, kv, step, table, n_heads: int, scale: float, window: int):
        """Grouped-query attention of the step's rows over the paged cache."""
        return ops.attn_plain(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window)

    def metadata(self, batch, mixers) -> dict:
        """Integer arrays the kernels want uploaded with the step (work lists); none here."""
        return {}

    def signature(self, batch, n_heads: int, n_kv_heads: int, head_dim: int, window: int):
        """What the kernels decide from the contexts' lengths (part of a recorded step's key)."""
        return ()


class TunedPagedAttention(PlainPagedAttention):
    def row_order(self, n_heads, n_kv_heads, head_dim, rotated_dims):
        if not rotated_dims:
            return None
        from .packing import rotary_paired_rows
        return rotary_paired_rows(n_heads, n_kv_heads, head_dim, rotated_dims)

    def project_rotate_store(self, x, w, step, table, angles, q_out, kv, n_heads, rotated_dims, writes):
        from . import tuned
        store = tuned.RopeStore(step.positions, step.tok_seq, table, angles, q_out, kv, n_heads, rotated_dims, writes)
        return tuned.gemm_rope_store(x, w, store, rt=self.rt)

    def attention(self, q, out, kv, step, table, n_heads, scale, window):
        from . import tuned
        return tuned.attention(self.rt, q, out, kv, step, table, n_heads, scale, window)

    def metadata(self, batch, mixers):
        """The rows and tiles of the batch, and for the single-row kernel the rows with splits of their
        own, one list per shape (blocks per row, window) among ``mixers``."""
        from . import tuned
        shapes = sorted({(tuned.decode_blocks_per_row(m.n_heads, m.n_kv_heads), m.window or 0) for m in mixers})
        return tuned.attention_metadata(batch, shapes)

    def signature(self, batch, n_heads, n_kv_heads, head_dim, window):
        from . import tuned
        return tuned.attention_splits(batch, n_heads, n_kv_heads, head_dim, window)


register_kernel_set("paged_attention", PlainPagedAttention, TunedPagedAttention)
