"""RMSNorm.  y = x * w * rsqrt(mean(x^2) + eps), sums in 32-bit
(crates/kernels-hip/src/kernels/rmsnorm_f16.cu:40-85); the fused form that first adds the
pending delta to the residual stream follows rmsnorm_f16_add_residual.cu."""
from __future__ import annotations

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
        return rt.gemm_add_norm(product.x, product.weight, resid, self.weight, self.eps)
