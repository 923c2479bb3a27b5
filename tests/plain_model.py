"""Plain, slow Mistral-dense decoder in numpy float64: whole sequences, no cache.

One function for each part.  Nothing here is shared with the product code under
``flambeau_amd/``: this file reads config.json and the safetensors file by
itself and is the oracle the engine is compared against.

Every formula cites the file of arte-fact/flambeau it was read from
(paths are relative to the reference checkout).
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------
# reading a model folder (independent of flambeau_amd.weights)
# --------------------------------------------------------------------------

_ST_DTYPES = {"F64": np.float64, "F32": np.float32, "F16": np.float16,
              "I32": np.int32, "I64": np.int64}


def _bf16_to_f64(raw: np.ndarray) -> np.ndarray:
    """bfloat16 bit patterns (uint16) to float64: bf16 is the top half of a float32."""
    return (raw.astype(np.uint32) << 16).view(np.float32).astype(F64)


def read_safetensors(path) -> dict:
    """All tensors of one safetensors file as float64 (integers stay integers)."""
    blob = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8:8 + hlen])
    data = memoryview(blob)[8 + hlen:]
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        shape = tuple(info["shape"])
        if info["dtype"] == "BF16":
            arr = _bf16_to_f64(np.frombuffer(data[lo:hi], dtype=np.uint16))
        else:
            arr = np.frombuffer(data[lo:hi], dtype=_ST_DTYPES[info["dtype"]])
            if arr.dtype.kind == "f":
                arr = arr.astype(F64)
        out[name] = arr.reshape(shape)
    return out


def read_model_dir(model_dir):
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    weights = read_safetensors(model_dir / "model.safetensors")
    return cfg, weights


def round_bf16(x: np.ndarray) -> np.ndarray:
    """Round float values to the nearest bfloat16 (ties to even), returned as float64."""
    f = np.ascontiguousarray(x, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).astype(F64).reshape(f.shape)


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def embedding(tokens, table):
    """h0[i,:] = E[token[i],:], no scaling; a token >= vocab is an error.

    crates/forward/src/core/composites/embed.rs:26-62 (bounds check :27-31).
    """
    tokens = np.asarray(tokens, dtype=np.int64)
    if tokens.size and (tokens.min() < 0 or tokens.max() >= table.shape[0]):
        raise ValueError("token id outside the vocabulary")
    return table[tokens].astype(F64)


def rmsnorm(x, weight, eps):
    """y = x * w / sqrt(mean(x^2) + eps): eps inside the root, added to the mean.

    crates/kernels-hip/src/kernels/rmsnorm_f16.cu:40-85
    (mean_sq = total/k; rsqrt = 1/sqrtf(mean_sq + eps); y = v*w*rsqrt);
    CPU form crates/model-ops/src/ops/rmsnorm.rs:204-217.
    """
    x = np.asarray(x, dtype=F64)
    mean_sq = (x * x).sum(axis=-1, keepdims=True) / x.shape[-1]
    return x / np.sqrt(mean_sq + eps) * np.asarray(weight, dtype=F64)


def linear(x, w):
    """y[n,out] = sum_k x[n,k] W[out,k]; W is [out_features, in_features], no bias.

    crates/kernels-hip/src/kernels/dense_gemv_f16_f16.cu:27-33 (w[n_rows,k]);
    crates/forward/src/loader/dense_attn.rs:108-147 (n_rows=out, n_cols=in);
    no bias field exists: crates/forward/src/ctx.rs:351-411.
    """
    return np.asarray(x, dtype=F64) @ np.asarray(w, dtype=F64).T


def rope_neox(x, positions, theta, rotated_dims=None):
    """Split-half rotation of x[n, heads, hd] by absolute position.

    pair i in [0, rot/2): f_i = theta^(-2i/rot); phi = pos*f_i;
    (x[i], x[i+rot/2]) <- (x[i]cos - x[i+rot/2]sin, x[i]sin + x[i+rot/2]cos).
    crates/kernels-hip/src/kernels/rope_neox_partial_f16.cu:37-52;
    CPU form crates/model-ops/src/ops/rope.rs:120-148.  Mistral rotates the
    whole head (rotated_dims = head_dim).
    """
    x = np.array(x, dtype=F64, copy=True)
    n, heads, hd = x.shape
    rot = hd if rotated_dims is None else rotated_dims
    half = rot // 2
    i = np.arange(half, dtype=F64)
    inv_freq = 1.0 / np.power(F64(theta), 2.0 * i / rot)
    ang = np.asarray(positions, dtype=F64)[:, None] * inv_freq[None, :]   # [n, half]
    c = np.cos(ang)[:, None, :]
    s = np.sin(ang)[:, None, :]
    lo = x[:, :, :half].copy()
    hi = x[:, :, half:rot].copy()
    x[:, :, :half] = lo * c - hi * s
    x[:, :, half:rot] = lo * s + hi * c
    return x


def attention(q, k, v, positions, scale, window=0, key_positions=None):
    """Causal grouped-query attention over one whole sequence.

    q[m, nh, hd] are queries at absolute positions ``positions``; k/v[n, nkv, hd] are the keys
    and values of the whole sequence at ``key_positions`` (the same places as the queries unless
    given: a caller that wants the output at a few rows only passes those rows' queries).
    kv_head = q_head // (nh // nkv); query at p sees keys t in
    [max(0, p-W+1), p] (W = 0: [0, p]); s_t = (q.k_t)*scale, scale applied after
    the dot; o = sum softmax(s)_t v_t over the visible keys only.
    crates/kernels-hip/src/kernels/attention_prefill_f16.cu:50-51 (head map),
    :58-71 (limit and window start), :89-133 (scores, softmax, PV);
    window counts keys including the query's own: crates/ops/tests/swa_softcap_parity.rs:243;
    default scale 1/sqrt(hd): crates/forward/src/core/composites/standard_attn.rs:418-420.

    Queries are taken 256 at a time, each batch against the keys that any of its queries sees, so that
    no score matrix is larger than 256 x n (the arithmetic per query is the same).
    """
    q = np.asarray(q, dtype=F64)
    k = np.asarray(k, dtype=F64)
    v = np.asarray(v, dtype=F64)
    positions = np.asarray(positions, dtype=np.int64)
    key_positions = positions if key_positions is None else np.asarray(key_positions, dtype=np.int64)
    m, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    lo = np.maximum(0, positions - window + 1) if window > 0 else np.zeros_like(positions)
    out = np.zeros((m, nh, v.shape[2]), dtype=F64)
    for a in range(0, m, 256):
        b = min(m, a + 256)
        near = np.nonzero((key_positions >= lo[a:b].min()) & (key_positions <= positions[a:b].max()))[0]
        kp = key_positions[near]
        # visible[i, t]: key t lies in [max(0, p_i - W + 1), p_i]
        visible = (kp[None, :] >= lo[a:b, None]) & (kp[None, :] <= positions[a:b, None])
        for h in range(nh):
            g = h // group
            s = (q[a:b, h, :] @ k[near, g, :].T) * scale
            s = np.where(visible, s, -np.inf)              # keys outside the range take no part
            s = s - s.max(axis=1, keepdims=True)
            w = np.exp(s)
            w = w / w.sum(axis=1, keepdims=True)
            out[a:b, h, :] = w @ v[near, g, :]
    return out


def silu(x):
    """silu(g) = g / (1 + exp(-g)).  crates/kernels-hip/src/kernels/swiglu_f32_to_f16.cu:21-23."""
    x = np.asarray(x, dtype=F64)
    return x / (1.0 + np.exp(-x))


def swiglu_mlp(x, w_gate, w_up, w_down):
    """d = (silu(x Wg^T) * (x Wu^T)) Wd^T.

    crates/forward/src/core/composites/dense_ffn.rs:116-137 (gate, up), :143 (SwiGLU),
    :176-186 (down).
    """
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


def default_scale(hd: int) -> float:
    """Score scale when the weights give none: 1 / sqrt(head_dim).
    crates/forward/src/core/composites/standard_attn.rs:418-420 ((head_dim as f32).sqrt().recip())."""
    return 1.0 / math.sqrt(hd)


def attention_mixer(x, w, prefix, positions, nh, nkv, hd, theta, window, rows=None):
    """Q/K/V projections, rotation of Q and K (not V), attention, output projection.

    crates/forward/src/core/composites/standard_attn.rs:198-286 (projections),
    :356-397 (rotation of Q and K), :1289-1301 (output projection).
    ``rows``: the output at these rows only (their queries against everyone's keys and values).
    """
    n = x.shape[0]
    positions = np.asarray(positions, dtype=np.int64)
    at = np.arange(n) if rows is None else np.asarray(rows, dtype=np.int64)
    q = linear(x[at], w[prefix + "q_proj.weight"]).reshape(len(at), nh, hd)
    k = linear(x, w[prefix + "k_proj.weight"]).reshape(n, nkv, hd)
    v = linear(x, w[prefix + "v_proj.weight"]).reshape(n, nkv, hd)
    q = rope_neox(q, positions[at], theta)
    k = rope_neox(k, positions, theta)
    o = attention(q, k, v, positions[at], default_scale(hd), window, key_positions=positions)
    return linear(o.reshape(len(at), nh * hd), w[prefix + "o_proj.weight"])


def config_numbers(cfg: dict) -> dict:
    """The numbers a Mistral config.json gives, with the defaults the format has."""
    nh = cfg["num_attention_heads"]
    return dict(
        H=cfg["hidden_size"], L=cfg["num_hidden_layers"], nh=nh,
        nkv=cfg.get("num_key_value_heads") or nh,
        hd=cfg.get("head_dim") or cfg["hidden_size"] // nh,
        I=cfg["intermediate_size"], V=cfg["vocab_size"], eps=cfg["rms_norm_eps"],
        theta=(cfg.get("rope_parameters") or {}).get("rope_theta") or cfg.get("rope_theta", 10000.0),
        window=cfg.get("sliding_window") or 0,
        tied=bool(cfg.get("tie_word_embeddings", False)),
        layer_types=cfg.get("layer_types"),
    )


def layer_window(c: dict, layer: int) -> int:
    """The window of one layer: ``sliding_window`` everywhere, unless ``layer_types`` names the layer
    "full_attention" (a per-layer switch as in crates/models/gemma4-v2/src/config.rs:124-138, where a
    per-layer pattern says which layers have the window)."""
    lt = c["layer_types"]
    if lt is None or lt[layer] == "sliding_attention":
        return c["window"]
    return 0


def forward(cfg: dict, w: dict, tokens, positions=None, keep_layers=None, rows=None) -> np.ndarray:
    """Logits [n, vocab] of one whole sequence (``rows``: only at these places, [len(rows), vocab]).

    for l: x += Attn(Norm1(x)); x += MLP(Norm2(x)); logits = Head(NormF(x)).
    crates/forward/README.md:28-40; crates/models/qwen35-v2/src/model.rs:19-50;
    final norm and head crates/forward/src/core/composites/output_head.rs:41-100;
    tied head = the embedding table again, crates/models/qwen35-v2/src/loader.rs:218-223.
    """
    c = config_numbers(cfg)
    n = len(tokens)
    if positions is None:
        positions = np.arange(n)
    x = embedding(tokens, w["model.embed_tokens.weight"])
    layers = list(range(c["L"]) if keep_layers is None else keep_layers)
    picked = None if rows is None else np.asarray(rows, dtype=np.int64)
    for i, l in enumerate(layers):
        p = f"model.layers.{l}."
        a = rmsnorm(x, w[p + "input_layernorm.weight"], c["eps"])
        # the last layer's output is needed at the wanted rows only: their queries against all keys
        only = picked if i == len(layers) - 1 else None
        mixed = attention_mixer(a, w, p + "self_attn.", positions, c["nh"], c["nkv"], c["hd"],
                                c["theta"], layer_window(c, l), rows=only)
        if only is not None:
            x, picked = x[only], None
        x = x + mixed
        b = rmsnorm(x, w[p + "post_attention_layernorm.weight"], c["eps"])
        x = x + swiglu_mlp(b, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])
    if picked is not None:
        x = x[picked]
    f = rmsnorm(x, w["model.norm.weight"], c["eps"])
    head = w["model.embed_tokens.weight"] if c["tied"] else w["lm_head.weight"]
    return linear(f, head)


def greedy_generate(cfg, w, prompt, n_new):
    """Argmax decoding by running the whole sequence again for every token."""
    toks = list(prompt)
    for _ in range(n_new):
        logits = forward(cfg, w, toks)
        toks.append(int(np.argmax(logits[-1])))
    return toks[len(prompt):]


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------

_M64 = (1 << 64) - 1


def _rotl(x, k):
    return ((x << k) | (x >> (64 - k))) & _M64


class Xoshiro:
    """xoshiro256** seeded through SplitMix64; next_f32 = (u64 >> 40) / 2^24.

    crates/runtime/src/sampling.rs:116-149.
    """

    def __init__(self, seed: int):
        x = (seed + 0x9E3779B97F4A7C15) & _M64
        s = []
        for _ in range(4):
            x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M64
            x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M64
            s.append(x ^ (x >> 31))
        if s == [0, 0, 0, 0]:
            s[0] = 1
        self.s = s

    def next_u64(self) -> int:
        s = self.s
        result = (_rotl((s[1] * 5) & _M64, 7) * 9) & _M64
        t = (s[1] << 17) & _M64
        s[2] ^= s[0]
        s[3] ^= s[1]
        s[1] ^= s[2]
        s[0] ^= s[3]
        s[2] ^= t
        s[3] = _rotl(s[3], 45)
        return result

    def next_f32(self) -> float:
        return float(np.float32(self.next_u64() >> 40) * np.float32(1.0 / (1 << 24)))


def apply_penalties(logits, history, repetition_penalty=1.0, presence_penalty=0.0,
                    frequency_penalty=0.0):
    """Per token seen in history: l>0 ? l/rp : l*rp; l -= pp; l -= fp*count.

    crates/runtime/src/sampling.rs:575-606.
    """
    out = np.array(logits, dtype=np.float32, copy=True)
    counts = {}
    for t in history:
        counts[t] = counts.get(t, 0) + 1
    for tok, c in counts.items():
        if tok >= out.shape[0]:
            continue
        l = out[tok]
        if repetition_penalty != 1.0 and repetition_penalty > 0.0:
            l = l / np.float32(repetition_penalty) if l > 0 else l * np.float32(repetition_penalty)
        if presence_penalty != 0.0:
            l = l - np.float32(presence_penalty)
        if frequency_penalty != 0.0:
            l = l - np.float32(frequency_penalty) * np.float32(c)
        out[tok] = l
    return out


def sample(logits, rng: Xoshiro, temperature=0.0, top_k=None, top_p=None, min_p=None,
           history=(), repetition_penalty=1.0, presence_penalty=0.0, frequency_penalty=0.0,
           logit_bias=None) -> int:
    """Penalties, bias, then argmax (temperature <= 0) or a multinomial draw.

    Order: crates/runtime/src/sampling.rs:306-335.  Argmax takes the first maximum
    (:486-496).  Stochastic path (:610-746): softmax of logits/T over the whole
    vocabulary; with a filter the candidates are sorted by falling probability,
    cut to top_k (2048 when only top_p/min_p is given), to the shortest prefix
    whose sum reaches top_p, and to those not below min_p * p_max; then
    u = rand * sum(kept) and the walk stops at the first entry where u <= 0.
    """
    l = apply_penalties(logits, history, repetition_penalty, presence_penalty, frequency_penalty)
    if logit_bias:
        for tok, b in logit_bias.items():
            if 0 <= tok < l.shape[0]:
                l[tok] += np.float32(b)
    if temperature <= 0.0:
        return int(np.argmax(l))
    inv_t = np.float32(1.0 / temperature)
    scaled = l * inv_t
    p = np.exp(scaled - scaled.max()).astype(np.float32)
    p = p / p.sum(dtype=np.float32)
    ids = np.arange(p.shape[0])
    if top_k is not None or top_p is not None or min_p is not None:
        order = np.argsort(-p, kind="stable")
        k_eff = top_k if top_k is not None else 2048
        order = order[:min(k_eff, order.shape[0])]
        end = order.shape[0]
        if top_p is not None and 0.0 < top_p < 1.0:
            cum = np.float32(0.0)
            prefix = 0
            for i in range(end):
                cum += p[order[i]]
                prefix = i + 1
                if cum >= top_p:
                    break
            end = prefix
        if min_p is not None and min_p > 0.0:
            thr = p[order[0]] * np.float32(min_p)
            drop = end
            for i in range(end):
                if p[order[i]] < thr:
                    drop = i
                    break
            end = max(drop, 1)
        ids = order[:end]
    kept = p[ids]
    total = np.float32(0.0)
    for pv in kept:                      # summed in order (sampling.rs:736), not pairwise
        total = np.float32(total + pv)
    u = np.float32(rng.next_f32()) * total
    for tok, pv in zip(ids, kept):
        u -= pv
        if u <= 0.0:
            return int(tok)
    return int(ids[-1])
