"""The full sampler on the host: penalties, bias, then argmax or a filtered multinomial draw.

Order and rules follow crates/runtime/src/sampling.rs:306-335 (order), :575-606 (penalties),
:168-176 (bias), :486-496 (argmax, first maximum), :610-746 (softmax over the whole vocabulary
at 1/T; candidates sorted by falling probability; top-k, with 2048 standing in when only top-p
or min-p is given; top-p prefix; min-p threshold; draw u = rand * sum(kept) and walk)."""
from __future__ import annotations

import numpy as np

from .params import SamplingParams
from .rng import Xoshiro256

TOP_K_AUTO_CAP = 2048


def penalised(logits: np.ndarray, params: SamplingParams, history) -> np.ndarray:
    out = np.array(logits, dtype=np.float32, copy=True)
    if params.has_penalties and len(history):
        toks, counts = np.unique(np.asarray(history, dtype=np.int64), return_counts=True)
        keep = toks < out.shape[0]
        toks, counts = toks[keep], counts[keep]
        l = out[toks]
        if params.repetition_penalty != 1.0:
            rp = np.float32(params.repetition_penalty)
            l = np.where(l > 0, l / rp, l * rp)
        if params.presence_penalty != 0.0:
            l = l - np.float32(params.presence_penalty)
        if params.frequency_penalty != 0.0:
            l = l - np.float32(params.frequency_penalty) * counts.astype(np.float32)
        out[toks] = l
    if params.logit_bias:
        for tok, b in params.logit_bias.items():
            if 0 <= int(tok) < out.shape[0]:
                out[int(tok)] += np.float32(b)
    return out


def sample_host(logits: np.ndarray, params: SamplingParams, history, rng: Xoshiro256) -> int:
    l = penalised(logits, params, history)
    if params.is_greedy:
        return int(np.argmax(l))
    scaled = l * np.float32(1.0 / params.temperature)
    p = np.exp(scaled - scaled.max()).astype(np.float32)
    s = p.sum(dtype=np.float32)
    if s > 0:
        p = p / s
    if params.has_filters:
        order = np.argsort(-p, kind="stable")
        k_eff = params.top_k if params.top_k is not None else TOP_K_AUTO_CAP
        order = order[:min(int(k_eff), order.shape[0])]
        probs = p[order]
        end = probs.shape[0]
        if params.top_p is not None and 0.0 < params.top_p < 1.0:
            cum = np.cumsum(probs, dtype=np.float32)
            hit = np.nonzero(cum >= np.float32(params.top_p))[0]
            end = int(hit[0]) + 1 if hit.size else end
        if params.min_p is not None and params.min_p > 0.0:
            below = np.nonzero(probs[:end] < probs[0] * np.float32(params.min_p))[0]
            if below.size:
                end = max(int(below[0]), 1)
        ids, kept = order[:end], probs[:end]
    else:
        ids, kept = None, p
    walk = np.cumsum(kept, dtype=np.float32)              # (the sum of the kept ones is added up in their order, as the walk is)
    u = np.float32(rng.next_f32()) * walk[-1]
    idx = int(np.searchsorted(walk, u, side="left"))      # first i with u - walk[i] <= 0
    idx = min(idx, kept.shape[0] - 1)
    return int(idx if ids is None else ids[idx])
