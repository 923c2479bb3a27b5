"""Grouped-query attention over the paged cache.

x -> Q, K, V (one joined matrix product) -> position encoding on Q and K -> K, V stored at
the tokens' positions -> softmax(Q K^T / sqrt(hd)) V over the keys
[max(0, p - window + 1), p] of the same request -> output projection.
(crates/forward/src/core/composites/standard_attn.rs:198-286 projections, :356-397
rotation, :485-500 paged store, :509-533 attention, :1289-1301 output projection; head map
kv_head = q_head / (n_heads / n_kv_heads), crates/kernels-hip/src/kernels/attention_prefill_f16.cu:50-51.)

This step's keys are stored before attention runs, so every query reads all its keys from the
cache and the same code serves whole prompts, portions and single decoded tokens.
"""
from __future__ import annotations

import math

import torch

from ..config.base import ConfigError
from ..kernels import ops
from ..kernels import paged_attention  # noqa: F401  (registers this mixer's kernel set)
from .base import MIXERS, POSITION_ENCODINGS, Mixer, PagedKVSpec, PartSpec, Product, TensorSpec


@MIXERS.register("paged_gqa_attention")
class PagedGQAAttention(Mixer):
    graph_safe = True
    lazy_input = True
    replayable = True

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: PartSpec, window: int = 0, scale: float | None = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key/value heads")
        if head_dim > ops.attention_max_head_dim():
            # refused when the model is built, not at its first step
            raise ConfigError(f"paged_gqa_attention: 'head_dim' {head_dim} is beyond what the attention kernels take "
                              f"(head sizes up to {ops.attention_max_head_dim()})")
        self.hidden_size = hidden_size
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.window = int(window or 0)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = POSITION_ENCODINGS.create(position)

    def cache_spec(self):
        return PagedKVSpec(self.n_kv_heads, self.head_dim, self.window)

    def subparts(self):
        return [self.position]

    def signature_group(self):
        return ("paged_gqa_attention", self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def step_signature(self, batch):
        """Into how many parts the kernels split the keys: all that this mixer decides from the
        contexts' lengths."""
        return self.kernels.signature(batch, self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def tensors(self):
        H, qw, kvw = self.hidden_size, self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
        return {"q.weight": TensorSpec((qw, H)), "k.weight": TensorSpec((kvw, H)),
                "v.weight": TensorSpec((kvw, H)), "o.weight": TensorSpec((H, qw))}

    @classmethod
    def step_metadata_for(cls, batch, mixers):
        """The work lists the attention kernels of the mixers' runtime want for the batch."""
        return mixers[0].kernels.metadata(batch, mixers) if mixers else {}

    def bind(self, weights, rt):
        self.rt = rt
        self.kernels = rt.kernels("paged_attention")
        w_qkv = torch.cat([weights["q.weight"], weights["k.weight"], weights["v.weight"]], dim=0)
        # Where the runtime's kernels want it, the rows of a rotated projection are put in an order in which the
        # product's own kernel can rotate (8 dims, their 8 partners, ...); the rotation kernel reads
        # that order too.
        rotary = self.position.rotary_parameters()
        order = self.kernels.row_order(self.n_heads, self.n_kv_heads, self.head_dim, rotary[0]) if rotary is not None else None
        self.paired = order is not None
        if self.paired:
            w_qkv = w_qkv[order.to(w_qkv.device)]
        self.w_qkv = rt.prepare_weight(w_qkv.contiguous())
        self.w_o = rt.prepare_weight(weights["o.weight"])
        self.position.bind({}, rt)

    def forward(self, x, step, cache):
        rt, n = self.rt, x.shape[0]
        nh, nkv, hd = self.n_heads, self.n_kv_heads, self.head_dim
        table = step.block_tables[cache.group]
        rotary = self.position.rotary_parameters()
        angles = self.position.rotary_table(rt, step) if rotary is not None and rotary[0] else None
        q = rt.buffer("attn_q", n, nh * hd)
        fused = False
        if self.paired and angles is not None:
            fused = self.kernels.project_rotate_store(x, self.w_qkv, step, table, angles, q, cache.kv, nh, rotary[0], cache.writes)
        if not fused:
            qkv = rt.buffer("attn_qkv", n, (nh + 2 * nkv) * hd, torch.float32)
            rt.gemm(x, self.w_qkv, qkv)
            if rotary is None:
                self.position.apply(qkv, step.positions, nh, nkv, hd)
                rotary = (0, 1.0)
            ops.rope_kv_write(qkv, step.positions, step.tok_seq, table, q, cache.kv, nh, rotary[0], rotary[1],
                              write_cache=cache.writes, table=angles, paired=self.paired)
        out = rt.buffer("attn_out", n, nh * hd)
        self.kernels.attention(q, out, cache.kv, step, table, nh, self.scale, self.window)
        return Product(out, self.w_o)
