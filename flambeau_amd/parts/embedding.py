"""Token embedding and output head.  Both are parts like the others: a model's description names
them by registry key (``EMBEDDINGS``, ``HEADS``), so a scaled embedding or a head with a soft cap is
another registered class, not a change to the model's code.  An embedding must offer ``weight``
(the table, for a tied head) and ``forward(tokens, out)``; a head ``bind(weights, rt,
embedding_table=...)`` and ``forward(x, max_rows) -> float32 logits``.

h0[i,:] = E[token[i],:], no scaling (crates/forward/src/core/composites/embed.rs:26-62);
logits = norm_f(x) Wlm^T in 32-bit, a tied head being the embedding table again
(crates/forward/src/core/composites/output_head.rs:41-100,
crates/models/qwen35-v2/src/loader.rs:218-223)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Part, TensorSpec


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size

    def tensors(self):
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size), "table")}

    def bind(self, weights, rt):
        self.rt = rt
        self.weight = weights["weight"]

    def forward(self, tokens, out):
        return ops.embed(self.weight, tokens, out)


@HEADS.register("linear_head")
class OutputHead(Part):
    replayable = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied = tied

    def tensors(self):
        return {} if self.tied else {"weight": TensorSpec((self.vocab_size, self.hidden_size))}

    def bind(self, weights, rt, embedding_table=None):
        self.rt = rt
        table = embedding_table if self.tied else weights["weight"]
        if table is None:
            raise ValueError("a tied output head needs the embedding table")
        # a tied head packs its own copy: the embedding keeps the row-major table for its gather
        self.weight = rt.prepare_weight(table)

    def forward(self, x, max_rows):
        logits = self.rt.buffer("logits", x.shape[0], self.vocab_size, torch.float32, max_rows=max_rows)
        self.rt.gemm(x, self.weight, logits)
        return logits
