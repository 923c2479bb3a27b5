"""Wrappers of the tuned bfloat16 kernels and the choice between them.

Every tuned kernel stands beside a plain one that computes the same thing; where a tuned
kernel does not take a shape (a K that is no multiple of 8, a head size beyond 256) the plain
kernel runs instead, so a size is never answered with a wrong result."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops
from .library import F, I, KernelError, P, call, register_signatures
from .ops import _check, dtype_code, stream_handle
from .packing import Weight, interleave_gate_up, pack_weight

register_signatures({
    "fl_gemm_skinny": [P, P, P, I, I, I, I, I, I, I, P],
    "fl_gemm_skinny_fused": [P, P, P, I, I, I, I, I, I, P, I, F, P, P, P, P, P],
    "fl_gemm_skinny_scale_parts": [I, I, I],
    "fl_gemm_skinny_rope": [P, P, I, I, I, P, I, F, P, P, P, I, P, P, P, I, I, I, I, I, I, I, P],
    "fl_gemm_tiled_rope": [P, P, I, I, I, P, I, F, P, P, P, I, P, P, P, I, I, I, I, I, I, I, P],
    "fl_gemm_tiled_rope_ex": [P, P, I, I, I, P, I, F, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, P],
    "fl_gemm_tiled_scaled": [P, P, P, P, I, I, I, I, I, I, P, I, F, P],
    "fl_gemm_tiled_residual": [P, P, P, I, I, I, P, P, P, P, P],
    "fl_gemm_tiled_parts": [I, I, I],
    "fl_gemm_tiled_residual_parts": [I, I, I],
    "fl_gemm_mid": [P, P, P, P, I, I, I, I, I, I, P],
    "fl_gemm_mid_splits": [I, I, I],
    "fl_gemm_mid_scaled": [P, P, P, P, I, I, I, I, I, I, P, I, F, P],
    "fl_gemm_mid_residual": [P, P, P, I, I, I, P, P, P, P, P],
    "fl_gemm_mid_parts": [I],
    "fl_gemm_mid_partials": [P, P, P, I, I, I, P, I, F, P],
    "fl_gemm_tiled_partials": [P, P, P, I, I, I, P, I, F, P],
    "fl_gemm_mid_ex": [P, P, P, P, I, I, I, I, I, I, P, I, F, I, I, P],
    "fl_gemm_tiled_ex": [P, P, P, P, I, I, I, I, I, I, P, I, F, I, I, P],
    "fl_gemm_tiled_residual_ex": [P, P, P, I, I, I, P, P, P, P, I, P],
    "fl_gemm_tiled": [P, P, P, P, I, I, I, I, I, I, P],
    "fl_gemm_tiled_splits": [I, I, I],
    "fl_gemm_tiled_shape": [I, I, I, I],
    "fl_attn_prefill": [P, P, P, P, I, P, P, I, I, I, I, I, I, F, I, I, P, P, I, P],
    "fl_attn_prefill_splits": [I, I, I, I, I],
    "fl_attn_prefill_heads": [I, I, I, I, I],
    "fl_attn_prefill_max_pages": [I],
    "fl_attn_prefill_takes": [I, I, I, I],
    "fl_attn_decode": [P, P, P, P, P, P, I, P, I, I, I, I, I, I, F, I, I, P],
    "fl_attn_decode_items": [P, P, P, P, P, P, I, P, I, I, I, I, I, I, F, I, P, I, P],
})

SKINNY_MAX_ROWS = 64     # rows the decode kernels take
SKINNY_BEST_ROWS = 16    # beyond one tile of tokens the kernel that shares x through LDS is faster


def _packed_size(n_rows: int, K: int) -> int:
    return (-(-n_rows // 16) * 16) * (-(-K // 32) * 32)


FUSED_NORM_MAX_ROWS = 16     # the skinny kernel's fusions with the norms around it take one tile of tokens


def mid_preferred(M: int, N: int, K: int) -> bool:
    """Whether the product that adds to the residual stream goes, at 9 to 16 rows, to the kernel that shares
    x through LDS although the skinny kernel takes it: from 9 rows on the skinny kernel fetches twice the x
    per byte of w, which a long K feels (measured, microseconds at 8 / 10 / 12 / 16 rows, the kernel that adds
    the K-splits included: 5120 x 32768 skinny 65 / 67 / 68 / 72, mid 57 throughout; 5120 x 14336 28 / 29 /
    30 / 31.5 against 27; 4096 x 14336 22.9 / 23.6 / 24.2 / 25.5 against 23.0 to 23.4).  Wide matrices with a
    short K stay with the skinny kernel, which shares x between two row groups from 9 rows on and is then as
    fast (65536 x 5120 at 16 rows: 107 us either way)."""
    if M <= 8 or K % 32 or K < 8192:
        return False
    nbytes = 2 * N * K
    return nbytes >= 140e6 or (M >= 13 and nbytes >= 100e6)


MID_PART_COLS = 4096         # columns per partial sum of squares that gemm_mid_residual leaves
MID_SCALE_PARTS = 4096       # parts the row scale of gemm_mid can add (up to 4 cost nothing, more a short loop before the product)


@dataclass
class NormedRows:
    """Rows ``norm(r)`` that exist only in factors: ``xg = bf16(r * g)`` (g = the norm's weight)
    and ``ssq[m, p]``, the sum of ``r[m]^2`` in parts, so that ``norm(r)[m] = xg[m] * rsqrt(sum_p
    ssq[m, p] / H + eps)``.  A product takes the factor out of its sum and applies it to its
    results (``gemm_skinny`` with ``row_scale``).  ``resid`` and ``weight`` are kept for kernels
    that want the rows themselves (``materialize``)."""
    xg: torch.Tensor
    ssq: torch.Tensor
    eps: float
    resid: torch.Tensor
    weight: torch.Tensor

    @property
    def shape(self):
        return self.xg.shape

    @property
    def dtype(self):
        return self.xg.dtype

    def materialize(self, rt):
        out = rt.buffer("normed_rows", self.xg.shape[0], self.xg.shape[1])
        return ops.rmsnorm(self.resid, self.weight, out, self.eps)


def skinny_parts(n_features: int) -> int:
    """Parts in which ``gemm_skinny_residual`` leaves the sums of squares of its N features."""
    return -(-n_features // 16)


def _row_scale_args(row_scale, M, K):
    if row_scale is None:
        return None, 0, 0.0
    parts = row_scale.ssq.shape[1]
    return _check(row_scale.ssq, "gemm.row_scale", torch.float32, (M, parts)), parts, float(row_scale.eps)


def gemm_skinny(x, w_packed, out, waves_per_block: int = 0, swiglu_rows: int = 0, row_scale: NormedRows | None = None):
    """``out = x @ w.T`` for up to 64 rows of x; ``w_packed`` = ``pack_weight(w)``, N rows taken
    from ``out``.  With ``swiglu_rows`` the packed matrix holds that many interleaved gate/up
    rows and ``out`` receives ``silu(gate) * up``.  With ``row_scale`` (then ``x`` is its ``xg``,
    at most 16 rows) every row of the product is scaled by the norm's factor first."""
    M, K = x.shape
    N = swiglu_rows or out.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    if row_scale is None:
        call("fl_gemm_skinny", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
             _check(out, "gemm.out", None, (M, None)), dtype_code(out.dtype), M, N, K, int(waves_per_block),
             1 if swiglu_rows else 0, out.shape[1], stream_handle())
        return out
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    call("fl_gemm_skinny_fused", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         _check(out, "gemm.out", None, (M, None)), dtype_code(out.dtype), M, N, K, 1 if swiglu_rows else 0,
         out.shape[1], ssq, parts, eps, None, None, None, None, stream_handle())
    return out


def gemm_skinny_residual(x, w_packed, resid, g, xg, ssq, eps: float, row_scale: NormedRows | None = None) -> NormedRows:
    """``resid += x @ w.T`` (float32, in place) for at most 16 rows, and the factors of the norm that
    follows: ``xg = bf16(resid * g)``, ``ssq[m, p]`` = sum of ``resid[m]^2`` over features 16 p .. 16 p + 15."""
    M, K = x.shape
    N = resid.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    in_ssq, parts, in_eps = _row_scale_args(row_scale, M, K)
    call("fl_gemm_skinny_fused", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         None, 0, M, N, K, 2, N, in_ssq, parts, in_eps, _check(resid, "gemm.resid", torch.float32, (M, N)),
         _check(g, "gemm.g", torch.float32, (N,)), _check(xg, "gemm.xg", torch.bfloat16, (M, N)),
         _check(ssq, "gemm.ssq", torch.float32, (M, skinny_parts(N))), stream_handle())
    return NormedRows(xg, ssq, float(eps), resid, g)


@dataclass
class RopeStore:
    """What the rotate-and-store epilogue of the joined q/k/v projection needs: where the tokens
    are (``positions``, ``tok_seq``, ``block_table``), the step's cosines and sines ``angles[n,
    rot / 2, 2]``, the buffer for the rotated q, and the layer's cache."""
    positions: torch.Tensor
    tok_seq: torch.Tensor
    block_table: torch.Tensor
    angles: torch.Tensor
    q_out: torch.Tensor
    cache: "ops.PagedLayerCache"
    n_heads: int
    rotated_dims: int
    write_cache: bool = True


def _rope_args(rs: RopeStore, M: int, N: int):
    c = rs.cache
    hd, nkv = c.head_dim, c.n_kv_heads
    if N != (rs.n_heads + 2 * nkv) * hd:
        raise KernelError(f"rope store: {N} features, expected {(rs.n_heads + 2 * nkv) * hd}")
    return (_check(rs.positions, "rope.positions", torch.int32, (M,)), _check(rs.tok_seq, "rope.tok_seq", torch.int32, (M,)),
            _check(rs.block_table, "rope.block_table", torch.int32, (None, None)), rs.block_table.shape[1],
            _check(rs.angles, "rope.angles", torch.float32, (M, rs.rotated_dims // 2, 2)),
            _check(rs.q_out, "rope.q_out", torch.bfloat16, (M, rs.n_heads * hd)),
            _check(c.pool, "rope.cache", torch.bfloat16), rs.n_heads, nkv, hd, c.page_size, c.n_pages,
            int(rs.rotated_dims), int(bool(rs.write_cache)))


def gemm_skinny_rope(x, w_packed, n_features: int, store: RopeStore, row_scale: NormedRows | None = None):
    """The joined q/k/v projection of at most 16 rows (rows of ``w`` in the order of
    ``rotary_paired_rows``): q is rotated into ``store.q_out``, k rotated and v as it is into the
    cache; nothing else is stored."""
    M, K = x.shape
    if w_packed.numel() != _packed_size(n_features, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{n_features}, {K}] matrix packs to {_packed_size(n_features, K)}")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    call("fl_gemm_skinny_rope", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         M, n_features, K, ssq, parts, eps, *_rope_args(store, M, n_features), stream_handle())
    return store.q_out


def gemm_rope_store(x, w: Weight, store: RopeStore, rt=None) -> bool:
    """The joined q/k/v projection with rotation and stores in the product's kernel, where a kernel
    for the shape exists; ``False`` if not (the caller then computes the product and calls the
    rotation kernel).  ``x`` may be ``NormedRows``."""
    if w.packed is None or store.rotated_dims % 16 or store.cache.head_dim % 16 or store.cache.pool.dtype != torch.bfloat16:
        return False
    M, K = x.shape
    if M <= FUSED_NORM_MAX_ROWS:
        x, scale = _rows_for(x, w, rt)
        gemm_skinny_rope(x, w.packed, w.rows, store, row_scale=scale)
        return True
    # many rows: the tiled product rotates and stores itself where its K is not split; where it is, it
    # leaves the splits apart and the rotation kernel adds them (at 7B sizes and 512 rows the product
    # with K split in two takes 45 us and the rotation kernel 13, the whole product in one kernel 82)
    if M > SKINNY_MAX_ROWS and K % 8 == 0:
        x, scale = _rows_for(x, w, rt)
        N = w.rows
        splits = gemm_tiled_splits(M, N, K)
        if splits == 1:
            gemm_tiled_rope(x, w.packed, N, store, row_scale=scale)
        else:
            parts = gemm_tiled_partials(x, w.packed, _split_workspace(rt, splits * M * N, x.device), N, row_scale=scale)
            ops.rope_kv_write(parts, store.positions, store.tok_seq, store.block_table, store.q_out, store.cache, store.n_heads,
                              store.rotated_dims, 0.0, write_cache=store.write_cache, table=store.angles, paired=True, parts=splits)
        return True
    if FUSED_NORM_MAX_ROWS < M <= SKINNY_MAX_ROWS and K % 32 == 0:
        # 17 to 64 rows: the product leaves its K-splits apart and the rotation kernel adds them
        x, scale = _rows_for(x, w, rt)
        N = w.rows
        splits = gemm_mid_splits(M, N, K)
        parts = gemm_mid_partials(x, w.packed, _split_workspace(rt, splits * M * N, x.device), N, row_scale=scale)
        ops.rope_kv_write(parts, store.positions, store.tok_seq, store.block_table, store.q_out, store.cache, store.n_heads,
                          store.rotated_dims, 0.0, write_cache=store.write_cache, table=store.angles, paired=True, parts=splits)
        return True
    return False


def gemm_tiled_rope(x, w_packed, n_features: int, store: RopeStore, row_scale: NormedRows | None = None, variant: int = 0):
    """``gemm_skinny_rope`` for many rows (shapes whose K is not split); ``variant`` as in ``gemm_tiled``."""
    M, K = x.shape
    if w_packed.numel() != _packed_size(n_features, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{n_features}, {K}] matrix packs to {_packed_size(n_features, K)}")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    args = (_check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
            M, n_features, K, ssq, parts, eps, *_rope_args(store, M, n_features))
    if variant:
        call("fl_gemm_tiled_rope_ex", *args, int(variant), stream_handle())
    else:
        call("fl_gemm_tiled_rope", *args, stream_handle())
    return store.q_out


def gemm_add_norm(rt, x, w: Weight, resid, norm_weight, eps: float):
    """``resid += x @ w.T`` with the norm that follows left in factors (``NormedRows``: ``resid * g`` in
    the compute dtype and the sums of squares in parts), by the product's own kernel or the kernel that
    adds its K-splits; ``None`` where no kernel takes the shape (the caller then runs product, addition
    and norm apart).  All shape rules of these kernels live here."""
    n, H = resid.shape
    if (w.packed is None or w.swiglu_cols or isinstance(x, NormedRows) or x.dtype != torch.bfloat16
            or x.shape[1] % 8 or H % 8):
        return None
    K = x.shape[1]
    xg = rt.buffer("normed_xg", n, H)
    if n <= FUSED_NORM_MAX_ROWS and not (H % 32 == 0 and mid_preferred(n, H, K)):
        ssq = rt.buffer("normed_ssq", n, skinny_parts(H), torch.float32)
        return gemm_skinny_residual(x, w.packed, resid, norm_weight, xg, ssq, eps)
    if n <= SKINNY_MAX_ROWS and K % 32 == 0 and H % 32 == 0:
        # 17 to 64 rows: the kernel that adds the K-splits of the product does it
        ssq = rt.buffer("normed_ssq_mid", n, mid_parts(H), torch.float32)
        workspace = _split_workspace(rt, gemm_mid_splits(n, H, K) * n * H, x.device)
        return gemm_mid_residual(x, w.packed, resid, norm_weight, xg, ssq, eps, workspace)
    if n > SKINNY_MAX_ROWS and H % 4 == 0:
        # many rows (a prompt portion): the tiled product's epilogue does it, or the kernel that adds its K-splits
        ssq = rt.buffer("normed_ssq_tiled", n, tiled_parts(n, H, K), torch.float32)
        splits = gemm_tiled_splits(n, H, K)
        workspace = _split_workspace(rt, splits * n * H, x.device) if splits > 1 else None
        return gemm_tiled_residual(x, w.packed, resid, norm_weight, xg, ssq, eps, workspace)
    return None


def gemm_mid_splits(M: int, N: int, K: int, waves: int = 0, splits: int = 0) -> int:
    from .library import load
    return load().fl_gemm_mid_splits_ex(M, N, K, waves, splits)


def gemm_mid(x, w_packed, out, workspace=None, swiglu_rows: int = 0, row_scale: NormedRows | None = None,
             waves: int = 0, splits: int = 0):
    """``out = x @ w.T`` for 17 to 64 rows of x (fewer are allowed) and K a multiple of 32: the
    waves of a block share x through LDS.  A narrow matrix splits K and needs ``workspace``
    (float32, ``gemm_mid_splits(M, N, K) * M * N`` values).  ``swiglu_rows`` and ``row_scale`` as in
    ``gemm_skinny``.  ``waves`` (4 or 8 per block) and ``splits`` fix what the kernel would choose
    (for tests and measurements)."""
    M, K = x.shape
    N = swiglu_rows or out.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    n_splits = 1 if swiglu_rows else gemm_mid_splits(M, N, K, waves, splits)
    if n_splits > 1 and (workspace is None or workspace.numel() < n_splits * M * N):
        raise KernelError(f"gemm_mid: [{M}, {N}, {K}] splits K {n_splits} ways and needs a workspace of {n_splits * M * N} floats")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    args = (_check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
            _check(out, "gemm.out", None, (M, None)),
            _check(workspace, "gemm.workspace", torch.float32) if workspace is not None else None,
            dtype_code(out.dtype), M, N, K, 1 if swiglu_rows else 0, out.shape[1], ssq, parts, eps)
    if waves or splits:
        call("fl_gemm_mid_ex", *args, int(waves), int(splits), stream_handle())
    else:
        call("fl_gemm_mid_scaled", *args, stream_handle())
    return out


def gemm_mid_partials(x, w_packed, workspace, n_features: int, row_scale: NormedRows | None = None):
    """The K-splits of ``x @ w.T`` (17 to 64 rows) left apart: returns ``[splits, M, N]`` float32 (a
    view of ``workspace``) for a kernel that adds them itself."""
    M, K = x.shape
    N = n_features
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    splits = gemm_mid_splits(M, N, K)
    if workspace is None or workspace.numel() < splits * M * N:
        raise KernelError(f"gemm_mid_partials: needs a workspace of {splits * M * N} floats")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    call("fl_gemm_mid_partials", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         _check(workspace, "gemm.workspace", torch.float32), M, N, K, ssq, parts, eps, stream_handle())
    return workspace[:splits * M * N].view(splits, M, N)


def mid_parts(n_features: int) -> int:
    """Parts in which ``gemm_mid_residual`` leaves the sums of squares of its N features."""
    return -(-n_features // MID_PART_COLS)


def gemm_mid_residual(x, w_packed, resid, g, xg, ssq, eps: float, workspace) -> NormedRows:
    """``gemm_skinny_residual`` for 17 to 64 rows: the kernel that adds the K-splits adds them to
    ``resid`` and leaves ``xg`` and ``ssq[m, p]`` (sums over 4096 features each).  ``workspace``:
    float32, ``gemm_mid_splits(M, N, K) * M * N`` values."""
    M, K = x.shape
    N = resid.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    if workspace is None or workspace.numel() < gemm_mid_splits(M, N, K) * M * N:
        raise KernelError(f"gemm_mid_residual: needs a workspace of {gemm_mid_splits(M, N, K) * M * N} floats")
    call("fl_gemm_mid_residual", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         _check(workspace, "gemm.workspace", torch.float32), M, N, K, _check(resid, "gemm.resid", torch.float32, (M, N)),
         _check(g, "gemm.g", torch.float32, (N,)), _check(xg, "gemm.xg", torch.bfloat16, (M, N)),
         _check(ssq, "gemm.ssq", torch.float32, (M, mid_parts(N))), stream_handle())
    return NormedRows(xg, ssq, float(eps), resid, g)


def gemm_tiled_splits(M: int, N: int, K: int, splits: int = 0) -> int:
    from .library import load
    return load().fl_gemm_tiled_splits_ex(M, N, K, splits)


def gemm_tiled(x, w_packed, out, workspace=None, swiglu_rows: int = 0, row_scale: NormedRows | None = None,
               variant: int = 0, splits: int = 0):
    """``out = x @ w.T`` for many rows of x.  A shape whose grid would not fill the chip splits K
    and needs ``workspace`` (float32, ``gemm_tiled_splits(M, N, K) * M * N`` values).  With
    ``swiglu_rows`` and ``row_scale`` see ``gemm_skinny``.  ``variant`` (block shape: 3 = 256 features x
    128 tokens, 7 = 192 x 128, 8 = 128 x 128, 10 = 256 x 256, 6 = 128 x 256) and ``splits`` fix what the kernel would
    choose (for tests and measurements)."""
    M, K = x.shape
    N = swiglu_rows or out.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    n_splits = 1 if swiglu_rows else gemm_tiled_splits(M, N, K, splits)
    if n_splits > 1 and (workspace is None or workspace.numel() < n_splits * M * N):
        raise KernelError(f"gemm_tiled: [{M}, {N}, {K}] splits K {n_splits} ways and needs a workspace of {n_splits * M * N} floats")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    args = (_check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
            _check(out, "gemm.out", None, (M, None)),
            _check(workspace, "gemm.workspace", torch.float32) if workspace is not None else None,
            dtype_code(out.dtype), M, N, K, 1 if swiglu_rows else 0, out.shape[1], ssq, parts, eps)
    if variant or splits:
        call("fl_gemm_tiled_ex", *args, int(variant), int(splits), stream_handle())
    else:
        call("fl_gemm_tiled_scaled", *args, stream_handle())
    return out


def gemm_tiled_partials(x, w_packed, workspace, n_features: int, row_scale: NormedRows | None = None):
    """``gemm_mid_partials`` for many rows: the K-splits of ``x @ w.T`` as ``[gemm_tiled_splits(M, N, K),
    M, N]`` float32 (a view of ``workspace``)."""
    M, K = x.shape
    N = n_features
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    splits = gemm_tiled_splits(M, N, K)
    if workspace is None or workspace.numel() < splits * M * N:
        raise KernelError(f"gemm_tiled_partials: needs a workspace of {splits * M * N} floats")
    ssq, parts, eps = _row_scale_args(row_scale, M, K)
    call("fl_gemm_tiled_partials", _check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
         _check(workspace, "gemm.workspace", torch.float32), M, N, K, ssq, parts, eps, stream_handle())
    return workspace[:splits * M * N].view(splits, M, N)


def tiled_parts(M: int, n_features: int, K: int, variant: int = 0) -> int:
    """Parts in which ``gemm_tiled_residual`` leaves the sums of squares of its N features."""
    from .library import load
    if variant and gemm_tiled_splits(M, n_features, K) == 1:
        return load().fl_gemm_tiled_parts_ex(M, n_features, K, variant)
    return load().fl_gemm_tiled_residual_parts(M, n_features, K)


def gemm_tiled_residual(x, w_packed, resid, g, xg, ssq, eps: float, workspace=None, variant: int = 0) -> NormedRows:
    """``gemm_skinny_residual`` for many rows: ``ssq[m, p]`` = sums over the tiles of features where K
    is not split, else over 4096 features each (the kernel that adds the K-splits does it then and
    needs ``workspace``: float32, ``gemm_tiled_splits(M, N, K) * M * N`` values)."""
    M, K = x.shape
    N = resid.shape[1]
    if w_packed.numel() != _packed_size(N, K):
        raise KernelError(f"gemm.w: packed matrix of {w_packed.numel()} values, a [{N}, {K}] matrix packs to {_packed_size(N, K)}")
    splits = gemm_tiled_splits(M, N, K)
    if splits > 1 and (workspace is None or workspace.numel() < splits * M * N):
        raise KernelError(f"gemm_tiled_residual: [{M}, {N}, {K}] splits K {splits} ways and needs a workspace of {splits * M * N} floats")
    args = (_check(x, "gemm.x", torch.bfloat16, (M, K)), _check(w_packed, "gemm.w", torch.bfloat16),
            _check(workspace, "gemm.workspace", torch.float32) if workspace is not None else None,
            M, N, K, _check(resid, "gemm.resid", torch.float32, (M, N)), _check(g, "gemm.g", torch.float32, (N,)),
            _check(xg, "gemm.xg", torch.bfloat16, (M, N)),
            _check(ssq, "gemm.ssq", torch.float32, (M, tiled_parts(M, N, K, variant))))
    if variant:
        call("fl_gemm_tiled_residual_ex", *args, int(variant), stream_handle())
    else:
        call("fl_gemm_tiled_residual", *args, stream_handle())
    return NormedRows(xg, ssq, float(eps), resid, g)


def _rows_for(x, w: Weight, rt):
    """``x`` and its row scale for a product with ``w``: factored rows stay factored where the
    skinny kernel runs, else the rows are made."""
    if not isinstance(x, NormedRows):
        return x, None
    M, K = x.shape
    if w.packed is not None and M <= FUSED_NORM_MAX_ROWS and K % 8 == 0:
        from .library import load
        parts = x.ssq.shape[1]
        if parts <= load().fl_gemm_skinny_scale_parts(w.packed_rows, K, parts):
            return x.xg, x
    if w.packed is not None and FUSED_NORM_MAX_ROWS < M <= SKINNY_MAX_ROWS and K % 32 == 0 \
            and x.ssq.shape[1] <= MID_SCALE_PARTS:
        return x.xg, x
    if w.packed is not None and M > SKINNY_MAX_ROWS and K % 8 == 0:
        return x.xg, x
    return x.materialize(rt), None


def _split_workspace(rt, n_floats: int, device):
    """Room for the partial sums of a product that splits K: one buffer for all shapes, in rows of
    4096 floats."""
    if rt is None:
        return torch.empty(n_floats, dtype=torch.float32, device=device)
    return rt.buffer("gemm_splitk", -(-n_floats // 4096), 4096, torch.float32, max_rows=1 << 20).view(-1)


def gemm(x, w: Weight, out, rt=None):
    """``out = x @ w.T`` with the best kernel that takes the shape; ``x`` may be ``NormedRows``."""
    x, scale = _rows_for(x, w, rt)
    M, K = x.shape
    if scale is not None and M <= FUSED_NORM_MAX_ROWS:
        return gemm_skinny(x, w.packed, out, row_scale=scale)
    if w.packed is not None and not w.swiglu_cols and x.dtype == torch.bfloat16 and K % 8 == 0:
        N = w.rows
        mid = SKINNY_BEST_ROWS < M <= SKINNY_MAX_ROWS and K % 32 == 0
        if M <= SKINNY_MAX_ROWS and not mid:
            return gemm_skinny(x, w.packed, out)
        splits = gemm_mid_splits(M, N, K) if mid else gemm_tiled_splits(M, N, K)
        workspace = _split_workspace(rt, splits * M * N, x.device) if splits > 1 else None
        if mid:
            return gemm_mid(x, w.packed, out, workspace, row_scale=scale)
        return gemm_tiled(x, w.packed, out, workspace, row_scale=scale)
    if w.rowmajor is None:
        raise KernelError(f"gemm: no kernel for {M} rows of a packed [{w.rows}, {w.cols}] matrix")
    return ops.gemm_plain(x, w.rowmajor, out)


def gemm_swiglu(x, w: Weight, out, rt):
    """``out = silu(x Wg^T) * (x Wu^T)``; ``w`` comes from ``prepare_gate_up``; ``x`` may be ``NormedRows``."""
    x, scale = _rows_for(x, w, rt)
    M, K = x.shape
    if scale is not None and w.swiglu_cols:
        kernel = gemm_skinny if M <= FUSED_NORM_MAX_ROWS else (gemm_mid if M <= SKINNY_MAX_ROWS else gemm_tiled)
        return kernel(x, w.packed, out, swiglu_rows=w.packed_rows, row_scale=scale)
    if scale is not None:
        x = scale.materialize(rt)
    if w.packed is not None and w.swiglu_cols and x.dtype == torch.bfloat16 and K % 8 == 0:
        if SKINNY_BEST_ROWS < M <= SKINNY_MAX_ROWS and K % 32 == 0:
            return gemm_mid(x, w.packed, out, swiglu_rows=w.packed_rows)
        if M <= SKINNY_MAX_ROWS:
            return gemm_skinny(x, w.packed, out, swiglu_rows=w.packed_rows)
        return gemm_tiled(x, w.packed, out, swiglu_rows=w.packed_rows)
    gu = rt.buffer("ffn_gate_up", M, w.rows, torch.float32)
    ops.gemm_plain(x, w.rowmajor, gu)
    return ops.silu_mul(gu, out)


def prepare_weight(w: torch.Tensor) -> Weight:
    """The form of a weight matrix the tuned path wants: packed tiles when the kernels take the
    shape (the row-major matrix is dropped then), else row-major for the plain kernel."""
    N, K = w.shape
    if w.dtype == torch.bfloat16 and K % 8 == 0:
        return Weight(N, K, packed=pack_weight(w), packed_rows=N)
    return Weight(N, K, rowmajor=w)


def prepare_gate_up(gate: torch.Tensor, up: torch.Tensor) -> Weight:
    I, K = gate.shape
    if gate.dtype == torch.bfloat16 and K % 8 == 0:
        inter = interleave_gate_up(gate, up)
        return Weight(2 * I, K, packed=pack_weight(inter), packed_rows=inter.shape[0], swiglu_cols=I)
    return Weight(2 * I, K, rowmajor=torch.cat([gate, up], dim=0).contiguous())


# Rows of portions up to this length are treated as single query rows by the split-K kernel;
# longer portions go to the tiled prefill kernel.
SHORT_PORTION = 8
DECODE_UNITS = 256                   # compute units of the device (``set_units``; an MI355X has 256)
DECODE_TARGET_BLOCKS = 512           # two blocks per compute unit
DECODE_EVEN_BLOCKS = 256             # one per unit: enough when all rows have about the same number of keys
DECODE_MIN_KEYS_PER_SPLIT = 128
DECODE_MAX_SPLITS = 64


PREFILL_TILE = 64        # query tokens per block of the tiled kernel


def set_units(units: int) -> None:
    """Plan the attention kernels' blocks for a device of ``units`` compute units (the runtime says so
    when it starts; the library's own plans ask the device themselves)."""
    global DECODE_UNITS, DECODE_TARGET_BLOCKS, DECODE_EVEN_BLOCKS
    DECODE_UNITS, DECODE_TARGET_BLOCKS, DECODE_EVEN_BLOCKS = int(units), 2 * int(units), int(units)


def attention_metadata(batch, shapes=()) -> dict:
    """Work lists for the attention kernels of one batch: ``attn_rows`` = (row, position, request,
    0) of the rows that run as single queries (decode rows and rows of short portions);
    ``attn_tiles`` = (request, first row, rows, index of the first row among all rows of tiles) for
    every 64 rows of the longer portions.  For every ``(blocks per row, window)`` in ``shapes`` (blocks
    that the single-row kernel runs per row and split: kv heads x tiles of 16 query heads) a list
    ``attn_items/<blocks>/<window>`` of the same rows with splits of their own and a list
    ``attn_item_rows/<blocks>/<window>`` of where each row's items begin (``balanced_items``)."""
    import numpy as np
    rows, tiles = [], []
    n_tile_rows = 0
    for s, (q0, ql, p0) in enumerate(zip(batch.q_starts, batch.q_lens, batch.start_pos)):
        if ql <= SHORT_PORTION:
            rows += [(q0 + i, p0 + i, s, 0) for i in range(ql)]
        else:
            for off in range(0, ql, PREFILL_TILE):
                cnt = min(PREFILL_TILE, ql - off)
                tiles.append((s, q0 + off, cnt, n_tile_rows))
                n_tile_rows += cnt
    rows = np.asarray(rows, dtype=np.int32).reshape(-1, 4)
    out = {"attn_rows": rows, "attn_tiles": np.asarray(tiles, dtype=np.int32).reshape(-1, 4)}
    for per_row, window in shapes:
        items, firsts = balanced_items(rows, per_row, window)
        out[f"attn_items/{per_row}/{window}"], out[f"attn_item_rows/{per_row}/{window}"] = items, firsts
        # whether any row is split at all decides if the kernel that merges runs: a part of the step's signature
        batch.notes[("attn_rows_split", per_row, window)] = bool(firsts.shape[0] and int(firsts[:, 2].max()) > 1)
    return out


def decode_blocks_per_row(n_heads: int, n_kv_heads: int) -> int:
    return n_kv_heads * -(-(n_heads // n_kv_heads) // 16)


def decode_item_budget(n_rows: int, blocks_per_row: int) -> int:
    """Places in the list of items for ``n_rows`` single rows: four per row, and what gives the chip
    ``DECODE_TARGET_BLOCKS`` blocks at least.  Depends on the batch's shape only, so a recorded step
    keeps its grid while the contexts grow; places that a step does not use cost next to nothing
    (their blocks come last and end at once)."""
    return max(n_rows, min(max(DECODE_TARGET_BLOCKS // max(1, blocks_per_row), 4 * n_rows), n_rows * DECODE_MAX_SPLITS))


# What the single-row kernel costs on this chip, measured with 8 to 64 rows of 2,100 keys at 7B head sizes:
# a compute unit streams keys and values at about 30 GB/s whether one block or two share it, so a step
# takes as long as the unit with the most bytes (blocks go to the 256 units in turn), a block costs 1.5 us
# beside its bytes, the kernel that merges splits 4.7 us, and the chip as a whole gives 6.4 TB/s.
DECODE_UNIT_RATE = 30e9
DECODE_CHIP_RATE = 6.4e12
DECODE_BLOCK_US = 1.5
DECODE_MERGE_US = 4.7
DECODE_KEY_BYTES = 512             # keys and values of one kv head of 128 dims in bfloat16 (the constants' reference)


def even_splits(n_rows: int, blocks_per_row: int, keys: float, most: int) -> int:
    """Splits per row (1 .. ``most``) for ``n_rows`` rows of about ``keys`` keys each: the number that makes
    the unit with the most blocks finish first by the measured costs above.  17 to 32 rows of 2,100 keys:
    one (a block per row and kv head, nothing to merge: 35 us where two splits take 42); 16 rows: two; 40: three."""
    units = n_rows * max(1, blocks_per_row)
    if units <= DECODE_TARGET_BLOCKS // 8:
        # few rows: two blocks per unit (measured up to 8 rows: 1 % of a 7B decode step faster than one)
        return max(1, min(most, DECODE_TARGET_BLOCKS // units))
    row_us = keys * DECODE_KEY_BYTES / DECODE_UNIT_RATE * 1e6
    chip_us = units * keys * DECODE_KEY_BYTES / DECODE_CHIP_RATE * 1e6
    best, best_us = 1, None
    for s in range(1, max(1, min(most, DECODE_MAX_SPLITS)) + 1):
        per_unit = -(-units * s // DECODE_UNITS)
        us = max(per_unit * (row_us / s + DECODE_BLOCK_US), chip_us) + (DECODE_MERGE_US if s > 1 else 0.0)
        if best_us is None or us < best_us * 0.97:              # (more splits only where they pay)
            best, best_us = s, us
    return best


def balanced_items(rows, blocks_per_row: int, window: int = 0, budget: int | None = None):
    """``rows`` (row, position, request, 0) with splits of their own: every row gets splits in
    proportion to the keys it sees (a split of 128 keys at least, 64 splits at most), so that the blocks
    of a ragged batch take about equally long.  Returns ``(items, firsts)``: ``items`` = (row,
    position, request, split + 256 * splits), a row's splits one after the other, the list filled up
    to ``decode_item_budget`` with row -1; ``firsts`` = (row, index of the row's first item, its
    splits, 0), one per row, for the kernel that merges."""
    import numpy as np
    n = rows.shape[0]
    if budget is None:
        budget = decode_item_budget(n, blocks_per_row)
    items = np.full((budget, 4), -1, dtype=np.int32)
    firsts = np.zeros((n, 4), dtype=np.int32)
    if n == 0:
        return items, firsts
    keys = rows[:, 1].astype(np.int64) + 1
    if window:
        keys = np.minimum(keys, window)
    most = np.minimum(-(-keys // DECODE_MIN_KEYS_PER_SPLIT), DECODE_MAX_SPLITS)
    # Rows that cannot be split anyway (a split holds 128 keys at least: the rows that pad a batch of
    # fixed shape, requests that have just begun) take a place each and have no say in what follows.
    big = most > 1
    n_big, n_small = int(big.sum()), int(n - big.sum())
    splits = np.ones(n, dtype=np.int64)
    if n_big:
        kb, mb = keys[big], most[big]
        # How many places to use.  Rows of about one length: the same number of splits for every row (a row
        # with one split beside rows with two ends the kernel alone), chosen by what the blocks then cost
        # (``even_splits``).  A ragged batch: all places, since many short blocks spread over the units as
        # they finish (55 rows of 128 to 4,600 keys: 136 us with a place per row, 100 with two, 94 with four).
        room = budget - n_small
        ragged = int(kb.max()) * n_big > 1.5 * int(kb.sum())
        if ragged:
            use = room
        else:
            each = even_splits(n_big, blocks_per_row, float(kb.mean()), min(int(mb.min()), max(1, room // n_big)))
            use = n_big * each
        sb = np.clip(kb * use // max(int(kb.sum()), 1), 1, mb)
        # what rounding down and the caps left over goes to the rows whose splits are longest; what the
        # least of one split per row took too much comes from the rows whose splits are shortest
        left = use - int(sb.sum())
        while left > 0:
            free = sb < mb
            if not free.any():
                break
            take = np.argsort(-np.where(free, kb / sb, 0.0), kind="stable")[:left]
            take = take[free[take]]
            sb[take] += 1
            left -= take.size
        while left < 0:
            give = np.argsort(np.where(sb > 1, kb / sb, np.inf), kind="stable")[:-left]
            give = give[sb[give] > 1]
            sb[give] -= 1
            left += give.size
        splits[big] = sb
    first = np.concatenate(([0], np.cumsum(splits)[:-1]))
    which = np.repeat(np.arange(n), splits)
    total = int(splits.sum())
    items[:total, :3] = rows[which, :3]
    items[:total, 3] = (np.arange(total) - first[which]) + 256 * splits[which]
    firsts[:, 0], firsts[:, 1], firsts[:, 2] = rows[:, 0], first, splits
    return items, firsts


def decode_splits(n_items: int, n_kv_heads: int, group: int, max_ctx: int) -> int:
    """How many splits of the keys give the chip enough blocks without making a split shorter
    than a few chunks.  Depends on the batch's shape only (fixed for a captured graph)."""
    base = max(1, n_items * n_kv_heads * -(-group // 16))
    by_blocks = max(1, DECODE_TARGET_BLOCKS // base)
    by_keys = max(1, -(-max_ctx // DECODE_MIN_KEYS_PER_SPLIT))
    return int(min(by_blocks, by_keys, 64))


def attn_decode(q, out, cache, rows, table, n_heads, scale, window, n_split, part_o=None, part_ml=None, firsts=None):
    """Attention of single query rows; ``rows[i] = (row of q and out, position, index of the request's
    row in ``table``, 0)``, every row's keys in ``n_split`` parts; or, with ``n_split`` = 0, rows with
    splits of their own as ``balanced_items`` lists them, with its list ``firsts`` of where each row's
    items begin (``None``: no row has more than one split, nothing is merged)."""
    n = q.shape[0]
    hd = cache.head_dim
    n_items = rows.shape[0]
    hdp = -(-hd // 32) * 32
    if n_split > 1 or (n_split == 0 and firsts is not None):
        slots = n_items * n_heads * max(n_split, 1)
        if part_o is None or part_o.numel() < slots * hdp or part_ml is None or part_ml.numel() < slots * 2:
            raise KernelError("attn_decode: workspace too small for the splits")
    head = (_check(q, "attn.q", torch.bfloat16, (n, n_heads * hd)), _check(out, "attn.out", torch.bfloat16, (n, n_heads * hd)),
            _check(part_o, "attn.part_o", torch.float32) if part_o is not None else None,
            _check(part_ml, "attn.part_ml", torch.float32) if part_ml is not None else None,
            _check(cache.pool, "attn.cache", torch.bfloat16), _check(rows, "attn.rows", torch.int32, (n_items, 4)), n_items,
            _check(table, "attn.block_table", torch.int32, (None, None)), table.shape[1], n_heads, cache.n_kv_heads,
            hd, cache.page_size, cache.n_pages, float(scale), int(window))
    if n_split == 0:
        call("fl_attn_decode_items", *head, _check(firsts, "attn.firsts", torch.int32, (None, 4)) if firsts is not None else None,
             firsts.shape[0] if firsts is not None else 0, stream_handle())
    else:
        call("fl_attn_decode", *head, int(n_split), stream_handle())
    return out


def attn_prefill_splits(n_tiles: int, n_heads: int, n_kv_heads: int, head_dim: int, max_keys: int) -> int:
    """Into how many parts the tiled kernel wants the keys split for a batch of this shape (1: not
    at all; more when few tiles face a long context)."""
    from .library import load
    return load().fl_attn_prefill_splits(n_tiles, n_heads, n_kv_heads, head_dim, max_keys)


def attn_prefill_heads(n_tiles: int, n_heads: int, n_kv_heads: int, head_dim: int, max_keys: int) -> int:
    """Query heads per wave that the tiled kernel wants for a batch of this shape (``heads_per_wave`` of
    ``attn_prefill``; the splits of ``attn_prefill_splits`` go with it)."""
    from .library import load
    return load().fl_attn_prefill_heads(n_tiles, n_heads, n_kv_heads, head_dim, max_keys)


def attn_prefill(q, out, cache, tiles, positions, table, n_heads, scale, window, heads_per_wave: int = 0,
                 n_split: int = 1, part_o=None, part_ml=None):
    """Attention of the longer portions; ``tiles[i] = (request's row in ``table``, first row, rows,
    index of the first row among all rows of tiles)``.  With ``n_split`` > 1 the keys are split and
    merged; ``part_o`` / ``part_ml``: float32 workspaces of rows x heads x n_split x (head_dim rounded
    up to 32, and 2) values, rows = all rows of tiles."""
    n = q.shape[0]
    hd = cache.head_dim
    n_tiles = tiles.shape[0]
    if n_split > 1:
        n_rows = int(tiles[-1, 2] + tiles[-1, 3]) if isinstance(tiles, torch.Tensor) and not tiles.is_cuda else None
        hdp = -(-hd // 32) * 32
        if part_o is None or part_ml is None:
            raise KernelError("attn_prefill: splits need a workspace")
        if n_rows is not None and (part_o.numel() < n_rows * n_heads * n_split * hdp or part_ml.numel() < n_rows * n_heads * n_split * 2):
            raise KernelError("attn_prefill: workspace too small for the splits")
    call("fl_attn_prefill", _check(q, "attn.q", torch.bfloat16, (n, n_heads * hd)),
         _check(out, "attn.out", torch.bfloat16, (n, n_heads * hd)), _check(cache.pool, "attn.cache", torch.bfloat16),
         _check(tiles, "attn.tiles", torch.int32, (n_tiles, 4)), n_tiles,
         _check(positions, "attn.positions", torch.int32, (n,)),
         _check(table, "attn.block_table", torch.int32, (None, None)), table.shape[1], n_heads, cache.n_kv_heads, hd,
         cache.page_size, cache.n_pages, float(scale), int(window), int(heads_per_wave),
         _check(part_o, "attn.part_o", torch.float32) if part_o is not None else None,
         _check(part_ml, "attn.part_ml", torch.float32) if part_ml is not None else None, int(n_split), stream_handle())
    return out


def decode_supported(cache) -> bool:
    return cache.pool.dtype == torch.bfloat16 and cache.head_dim % 8 == 0 and cache.head_dim <= 256 \
        and cache.page_size % 8 == 0


def prefill_max_pages(head_dim: int) -> int:
    """Block-table entries per request that the tiled kernel takes (it keeps a request's table in LDS
    beside its ring of keys and values); the library is the one place that knows."""
    from .library import load
    return load().fl_attn_prefill_max_pages(int(head_dim))


def prefill_supported(cache, table, window: int = 0) -> bool:
    """Whether the tiled kernel takes this cache with block tables this wide (the library decides)."""
    from .library import load
    return cache.pool.dtype == torch.bfloat16 and bool(
        load().fl_attn_prefill_takes(cache.head_dim, cache.page_size, table.shape[1], int(window or 0)))


def attention_splits(batch, n_heads: int, n_kv_heads: int, head_dim: int, window: int, with_items: bool = True):
    """``(parts of the keys for the tiled kernel + 64 x its query heads per wave, parts for the single-row
    kernel)`` for a batch: everything that ``attention`` decides from the contexts' lengths (the rest
    follows from the batch's shape).
    ``with_items``: the single rows come with splits of their own (``balanced_items``), which are
    data of the step; all they decide here is whether any row is split at all (0 if so: the kernel
    that merges runs; -1 if not: it is left out)."""
    n_tiles = sum(-(-ql // PREFILL_TILE) for ql in batch.q_lens if ql > SHORT_PORTION)
    n_items = sum(ql for ql in batch.q_lens if ql <= SHORT_PORTION)
    p_split = n_split = 1
    if n_tiles:
        # few tiles before a long context: the keys are split too, so that the chip has blocks enough
        longest = batch.max_ctx_len if not window else min(batch.max_ctx_len, window + PREFILL_TILE)
        p_split = attn_prefill_splits(n_tiles, n_heads, n_kv_heads, head_dim, longest) \
            + 64 * attn_prefill_heads(n_tiles, n_heads, n_kv_heads, head_dim, longest)
    if n_items and not with_items:
        max_ctx = batch.ctx_bound or batch.max_ctx_len
        if window:
            max_ctx = min(max_ctx, window + 32)
        n_split = decode_splits(n_items, n_kv_heads, n_heads // n_kv_heads, max_ctx)
    if n_items and with_items:
        split = batch.notes.get(("attn_rows_split", decode_blocks_per_row(n_heads, n_kv_heads), window or 0), True)
        return p_split, (0 if split else -1)
    return p_split, n_split


def attention(rt, q, out, cache, step, table, n_heads, scale, window):
    """Attention of one batch with the tuned kernels: rows of short portions through the split-K
    kernel, longer portions through the tiled kernel.  A cache shape one of them does not take
    sends the whole batch to the plain kernel."""
    rows, tiles = step.extra.get("attn_rows"), step.extra.get("attn_tiles")
    batch = step.host
    if rows is None or tiles is None or not decode_supported(cache) or (tiles.shape[0] and not prefill_supported(cache, table, window)):
        return ops.attn_plain(q, out, cache, step.positions, step.tok_seq, table, n_heads, scale, window)
    items = step.extra.get(f"attn_items/{decode_blocks_per_row(n_heads, cache.n_kv_heads)}/{window or 0}")
    key = ("attention_splits", n_heads, cache.n_kv_heads, cache.head_dim, window)
    splits = step.scratch.get(key)
    if splits is None:
        splits = step.scratch[key] = attention_splits(batch, n_heads, cache.n_kv_heads, cache.head_dim, window,
                                                       with_items=items is not None)
    p_split, n_split = splits
    p_heads, p_split = p_split >> 6, p_split & 63
    if tiles.shape[0]:
        p_o = p_ml = None
        if p_split > 1:
            n_rows = sum(ql for ql in batch.q_lens if ql > SHORT_PORTION)
            hdp = -(-cache.head_dim // 32) * 32
            p_o = rt.buffer("attn_tile_part_o", n_rows * n_heads * p_split, hdp, torch.float32, max_rows=1 << 24)
            p_ml = rt.buffer("attn_tile_part_ml", n_rows * n_heads * p_split, 2, torch.float32, max_rows=1 << 24)
        attn_prefill(q, out, cache, tiles, step.positions, table, n_heads, scale, window, heads_per_wave=p_heads,
                     n_split=p_split, part_o=p_o, part_ml=p_ml)
    if rows.shape[0] and items is not None:
        # rows with splits of their own; the list's length follows from the number of rows alone
        # (a list with a place per row and no more: no row is ever split, nothing to merge)
        firsts = step.extra.get(f"attn_item_rows/{decode_blocks_per_row(n_heads, cache.n_kv_heads)}/{window or 0}")
        if items.shape[0] <= rows.shape[0] or n_split < 0:
            firsts = None                    # no row is split: every block writes its row itself
        part_o = part_ml = None
        if firsts is not None:
            hdp = -(-cache.head_dim // 32) * 32
            slots = items.shape[0] * n_heads
            part_o = rt.buffer("attn_part_o", slots, hdp, torch.float32, max_rows=1 << 24)
            part_ml = rt.buffer("attn_part_ml", slots, 2, torch.float32, max_rows=1 << 24)
        attn_decode(q, out, cache, items, table, n_heads, scale, window, 0, part_o, part_ml, firsts=firsts)
    elif rows.shape[0]:
        part_o = part_ml = None
        if n_split > 1:
            hdp = -(-cache.head_dim // 32) * 32
            slots = rows.shape[0] * n_heads * n_split
            cap = slots if batch.ctx_bound else max(slots, 4096 * n_heads)     # a fixed-shape step never grows
            part_o = rt.buffer("attn_part_o", slots, hdp, torch.float32, max_rows=cap)
            part_ml = rt.buffer("attn_part_ml", slots, 2, torch.float32, max_rows=cap)
        attn_decode(q, out, cache, rows, table, n_heads, scale, window, n_split, part_o, part_ml)
    return out
