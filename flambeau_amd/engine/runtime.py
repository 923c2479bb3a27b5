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
        lib = load()   # fails loudly when the kernel library cannot be built or loaded
        if bool(tuned) and dtype == torch.bfloat16:
            from ..kernels import tuned as tuned_kernels
            tuned_kernels.set_units(lib.fl_compute_units())
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
        self._kernel_sets: dict = {}

    def kernels(self, name: str):
        """The kernel set ``name`` in the form this runtime runs (``kernels/sets.py``): what a kind of
        part needs beyond matrix products.  The runtime knows no set by name; parts register theirs."""
        ks = self._kernel_sets.get(name)
        if ks is None:
            from ..kernels.sets import make_kernel_set
            ks = self._kernel_sets[name] = make_kernel_set(name, self)
        return ks

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

    def gemm_add_norm(self, x, w, resid, norm_weight, eps: float):
        """``resid += x @ w.T`` with the norm that follows left in factors, where a kernel does both
        (``kernels.tuned.gemm_add_norm``); ``None`` if none does: the caller adds and norms itself."""
        if not self.tuned:
            return None
        from ..kernels import tuned
        return tuned.gemm_add_norm(self, x, w, resid, norm_weight, eps)

    def gemm_swiglu(self, x, w, out):
        """``out = silu(x Wg^T) * (x Wu^T)``; ``w`` comes from ``prepare_gate_up``.  The tuned
        kernels apply the gate before they store; the plain path is a product and a gate kernel."""
        if self.tuned:
            from ..kernels import tuned
            return tuned.gemm_swiglu(x, w, out, self)
        gu = self.buffer("ffn_gate_up", x.shape[0], w.rows, torch.float32)
        ops.gemm_plain(x, w.rowmajor, gu)
        return ops.silu_mul(gu, out)
