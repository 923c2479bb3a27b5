"""RMSNorm.  y = x * w * rsqrt(mean(x^2) + eps), sums in 32-bit
(crates/kernels-hip/src/kernels/rmsnorm_f16.cu:40-85); the fused form that first adds the
pending delta to the residual stream follows rmsnorm_f16_add_residual.cu."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import NORMS, Norm, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    replayable = True

    def __init__(self, hidden_size: int, eps: float):
        self.hidden_size = hidden_size
        self.eps = eps

    def tensors(self):
        return {"weight": TensorSpec((self.hidden_size,), "vector32")}

    def bind(self, weights, rt):
        self.rt = rt
        self.weight = weights["weight"]

    def forward(self, x, out, delta=None, store_sum=False, rows=None):
        return ops.rmsnorm(x, self.weight, out, self.eps, delta=delta, store_sum=store_sum, rows=rows)

    def after_product(self, rt, resid, product):
        """Where a kernel for the shape exists the product's kernel adds its result to the stream and
        leaves the norm in factors: x * w in the compute dtype and the sums of squares in parts.
        The product that follows multiplies by rsqrt(mean + eps) itself: no norm kernel runs."""
        if not rt.tuned:
            return None
        from ..kernels import tuned
        n, H = resid.shape
        w, x = product.weight, product.x
        if (w.packed is None or w.swiglu_cols or isinstance(x, tuned.NormedRows) or x.dtype != torch.bfloat16
                or x.shape[1] % 8 or H % 8):
            return None
        K = x.shape[1]
        xg = rt.buffer("normed_xg", n, H)
        if n <= tuned.FUSED_NORM_MAX_ROWS:
            ssq = rt.buffer("normed_ssq", n, tuned.skinny_parts(H), torch.float32)
            return tuned.gemm_skinny_residual(x, w.packed, resid, self.weight, xg, ssq, self.eps)
        if n <= tuned.SKINNY_MAX_ROWS and K % 32 == 0 and H % 32 == 0:
            # 17 to 64 rows: the kernel that adds the K-splits of the product does it
            ssq = rt.buffer("normed_ssq_mid", n, tuned.mid_parts(H), torch.float32)
            workspace = tuned._split_workspace(rt, tuned.gemm_mid_splits(n, H, K) * n * H, x.device)
            return tuned.gemm_mid_residual(x, w.packed, resid, self.weight, xg, ssq, self.eps, workspace)
        if n > tuned.SKINNY_MAX_ROWS and H % 4 == 0:
            # many rows (a prompt portion): the tiled product's epilogue does it, or the kernel that adds its K-splits
            ssq = rt.buffer("normed_ssq_tiled", n, tuned.tiled_parts(n, H, K), torch.float32)
            splits = tuned.gemm_tiled_splits(n, H, K)
            workspace = tuned._split_workspace(rt, splits * n * H, x.device) if splits > 1 else None
            return tuned.gemm_tiled_residual(x, w.packed, resid, self.weight, xg, ssq, self.eps, workspace)
        return None
