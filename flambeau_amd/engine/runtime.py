"""The device context parts run in: dtype, activation buffers, matrix products.

All activation buffers are allocated once at ``max_batch_tokens`` rows and handed out as
row prefixes, so addresses never change between steps (a captured graph replays on the
same memory).  The reference does the same with its ``ScratchPool``
(crates/forward/src/core/scratch.rs:819-1058).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.library import KernelError, load


class Runtime:
    def __init__(self, device="cuda:0", dtype=torch.bfloat16, max_batch_tokens: int = 2048,
                 tuned: bool = True):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype must be float32 or bfloat16, got {dtype}")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("flambeau_amd runs on the GPU only: there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("flambeau_amd: no GPU visible to this process")
        torch.cuda.set_device(self.device)
        load()   # fails loudly when the kernel library cannot be built or loaded
        self.dtype = dtype
        # tuned kernels exist for bfloat16 only; the 32-bit path always runs the plain ones
        self.tuned = bool(tuned) and dtype == torch.bfloat16
        self.max_batch_tokens = int(max_batch_tokens)
        # rows per tile of the matrix kernels that take prompt portions (a scheduler that knows it
        # can fill whole tiles); the plain kernels have none
        self.row_granule = 128 if self.tuned else 1
        self._buffers: dict = {}
        self._views: dict = {}
        self._scope = ""
        self.generation = 0          # counts allocations of buffers: recorded launches name buffers by address

    # ------------------------------------------------------------ buffers
    def buffer(self, name: str, rows: int, cols: int, dtype=None, max_rows: int | None = None):
        """A ``[rows, cols]`` view of the buffer ``name``.  A buffer grows (to the next power of
        two of rows, never beyond its maximum) when a step needs more rows than any before."""
        dtype = dtype or self.dtype
        cap = max_rows if max_rows is not None else self.max_batch_tokens
        if rows > cap:
            raise KernelError(f"buffer '{name}': {rows} rows asked, at most {cap} allowed")
        key = (self._scope, name, cols, dtype)
        view = self._views.get((key, rows))             # (slicing a tensor costs a microsecond or two, a step asks 400 times)
        if view is not None:
            return view
        buf = self._buffers.get(key)
        if buf is None or buf.shape[0] < rows:
            size = min(cap, max(16, 1 << max(rows - 1, 0).bit_length()))
            buf = torch.empty((size, cols), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.generation += 1
            for k in [k for k in self._views if k[0] == key]:
                del self._views[k]
        view = self._views[(key, rows)] = buf[:rows]
        return view

    def scope(self, name: str):
        """Buffers asked for inside ``with rt.scope(name)`` are separate from all others (a
        captured graph keeps its own, which never move)."""
        rt = self

        class _Scope:
            def __enter__(self_inner):
                self_inner.prev, rt._scope = rt._scope, name
            def __exit__(self_inner, *exc):
                rt._scope = self_inner.prev
        return _Scope()

    def to_device(self, t: torch.Tensor, role: str) -> torch.Tensor:
        """A loaded tensor in the dtype its role asks for, on the device."""
        if role in ("matrix", "table"):
            want = self.dtype
        elif role == "vector32":
            want = torch.float32
        elif role == "int32":
            want = torch.int32
        else:
            raise ValueError(f"unknown tensor role '{role}'")
        return t.to(device=self.device, dtype=want).contiguous()

    # ------------------------------------------------------------ matrix products
    def prepare_weight(self, w: torch.Tensor):
        """A loaded matrix ``[out_features, in_features]`` in the form(s) the kernels of this
        runtime read: row-major for the plain kernels, packed tiles for the tuned ones."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.prepare_weight(w)
        from ..kernels.packing import Weight
        return Weight(w.shape[0], w.shape[1], rowmajor=w)

    def prepare_gate_up(self, gate: torch.Tensor, up: torch.Tensor):
        """Gate and up matrices of a gated feed-forward as one weight for ``gemm_swiglu``."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.prepare_gate_up(gate, up)
        from ..kernels.packing import Weight
        return Weight(2 * gate.shape[0], gate.shape[1], rowmajor=torch.cat([gate, up], dim=0).contiguous())

    def gemm(self, x, w, out):
        """``out = x @ w.T``; ``w`` comes from ``prepare_weight``."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.gemm(x, w, out, rt=self)
        return ops.gemm_plain(x, w.rowmajor, out)

    def gemm_rope_store(self, x, w, step, table, angles, q_out, kv, n_heads: int, rotated_dims: int, writes: bool) -> bool:
        """The joined q/k/v projection fused with rotation and the stores of q (into ``q_out``) and of
        the cache rows (into ``kv`` where ``writes``); the rows of ``w`` lie in ``rotary_row_order``,
        ``angles`` are the step's cosines and sines.  ``False`` if no kernel takes the shape: the
        caller then runs product and rotation apart."""
        if not self.tuned:
            return False
        from ..kernels import tuned
        store = tuned.RopeStore(step.positions, step.tok_seq, table, angles, q_out, kv, n_heads, rotated_dims, writes)
        return tuned.gemm_rope_store(x, w, store, rt=self)

    def gemm_add_norm(self, x, w, resid, norm_weight, eps: float):
        """``resid += x @ w.T`` with the norm that follows left in factors, where a kernel does both
        (``kernels.tuned.gemm_add_norm``); ``None`` if none does: the caller adds and norms itself."""
        if not self.tuned:
            return None
        from ..kernels import tuned
        return tuned.gemm_add_norm(self, x, w, resid, norm_weight, eps)

    def rotary_row_order(self, n_heads: int, n_kv_heads: int, head_dim: int, rotated_dims: int):
        """The order in which the rows of a joined q/k/v matrix have to lie for ``gemm_rope_store``
        (a permutation), or ``None`` where the kernels of this runtime read them as they are."""
        if not self.tuned or not rotated_dims:
            return None
        from ..kernels.packing import rotary_paired_rows
        return rotary_paired_rows(n_heads, n_kv_heads, head_dim, rotated_dims)

    def attention(self, q, out, kv, step, table, n_heads: int, scale: float, window: int):
        """Grouped-query attention of the step's rows over the paged cache."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.attention(self, q, out, kv, step, table, n_heads, scale, window)
        return ops.attn_plain(q, out, kv, step.positions, step.tok_seq, table, n_heads, scale, window)

    def attention_metadata(self, batch, mixers):
        """The attention kernels' work lists for a batch (integer arrays for the step's upload): the
        rows and tiles, and for the tuned single-row kernel the rows with splits of their own, one
        list per shape (blocks per row, window) among ``mixers``."""
        from ..kernels import tuned
        shapes = ()
        if self.tuned:
            shapes = sorted({(tuned.decode_blocks_per_row(m.n_heads, m.n_kv_heads), m.window or 0) for m in mixers})
        return tuned.attention_metadata(batch, shapes)

    def attention_splits(self, batch, n_heads: int, n_kv_heads: int, head_dim: int, window: int):
        """What the attention kernels of this runtime decide from the contexts' lengths (part of a
        recorded step's key); nothing for the plain kernels."""
        if not self.tuned:
            return ()
        from ..kernels import tuned
        return tuned.attention_splits(batch, n_heads, n_kv_heads, head_dim, window)

    def gemm_swiglu(self, x, w, out):
        """``out = silu(x Wg^T) * (x Wu^T)``; ``w`` comes from ``prepare_gate_up``.  The tuned
        kernels apply the gate before they store; the plain path is a product and a gate kernel."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.gemm_swiglu(x, w, out, self)
        gu = self.buffer("ffn_gate_up", x.shape[0], w.rows, torch.float32)
        ops.gemm_plain(x, w.rowmajor, gu)
        return ops.silu_mul(gu, out)
