"""Dense SwiGLU feed-forward: d = (silu(x Wg^T) * (x Wu^T)) Wd^T
(crates/forward/src/core/composites/dense_ffn.rs:116-186).  Gate and up matrices are
joined at load so that one matrix product feeds both and applies the gate before it stores."""
from __future__ import annotations

import torch

from .base import FEED_FORWARDS, FeedForward, Product, TensorSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    replayable = True
    lazy_input = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size

    def tensors(self):
        H, I = self.hidden_size, self.intermediate_size
        return {"gate.weight": TensorSpec((I, H)), "up.weight": TensorSpec((I, H)),
                "down.weight": TensorSpec((H, I))}

    def bind(self, weights, rt):
        self.rt = rt
        self.w_gate_up = rt.prepare_gate_up(weights["gate.weight"], weights["up.weight"])
        self.w_down = rt.prepare_weight(weights["down.weight"])

    def forward(self, x, step):
        rt, n, I = self.rt, x.shape[0], self.intermediate_size
        act = rt.buffer("ffn_act", n, I)
        rt.gemm_swiglu(x, self.w_gate_up, act)
        return Product(act, self.w_down)
