"""Throughput of the engine on one MI355X: decode tokens/s and prefill tokens/s.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Default run: Mistral-7B-v0.3 layer sizes, random weights, bfloat16, a batch of 8 requests
that each hold a 2,048-token prompt in the cache and decode greedily (context up to 4,096),
through the engine's own loop: scheduler, step function, device sampler.  One "step" is one
decode step of the whole batch.  Prints ONE JSON line; ``value`` is decoded tokens per second.
The same line carries the 2,048-token prefill, the decode step's memory roofline and decode at
batch 1 and 64.  Definitions follow the reference's (doc/PERF_MATRIX.md:5-8): prefill tok/s =
prompt tokens / time to first token, decode tok/s over the decode interval only.
"""
from __future__ import annotations

import argparse
import json
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# Mistral-7B-v0.3 sizes (the benchmark configuration)
CONFIG_7B = {
    "architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
    "num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "intermediate_size": 14336, "vocab_size": 32768, "rope_theta": 1e6,
    "sliding_window": None, "rms_norm_eps": 1e-5, "max_position_embeddings": 32768,
    "tie_word_embeddings": False,
}
PEAK_HBM = 8.0e12            # bytes/s, MI355X
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PROMPT_LEN = 2048
CONTEXT = 4096
PAGE = 16


def sizes(cfg, n_layers):
    H, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    I, V = cfg["intermediate_size"], cfg["vocab_size"]
    per_layer = (nh + 2 * nkv) * hd * H + H * nh * hd + 3 * I * H
    return dict(matrix_params=n_layers * per_layer, head_params=V * H,
                kv_values_per_token=n_layers * 2 * nkv * hd, nh=nh, hd=hd, n_layers=n_layers)


def decode_bytes(sz, batch, mean_ctx, el):
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    return (sz["matrix_params"] + sz["head_params"]) * el + batch * mean_ctx * sz["kv_values_per_token"] * el


def prefill_flops(sz, T):
    gemm = 2.0 * T * sz["matrix_params"] + 2.0 * sz["head_params"]
    attn = sz["n_layers"] * 2.0 * T * T * sz["hd"] * sz["nh"]       # causal: half of 4 T^2 hd nh
    return gemm + attn


def run_decode(model, batch, steps, warmup, dtype_name, seed=0):
    """Time ``steps`` decode steps of ``batch`` requests, each with a PROMPT_LEN prompt in the cache."""
    import numpy as np
    import torch
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    opt = EngineOptions(dtype=dtype_name, inflight_slots=batch, prefill_chunk_tokens=PROMPT_LEN,
                        page_size=PAGE, ctx_cap=CONTEXT, paged_kv=batch * CONTEXT // PAGE)
    eng = LLMEngine(model, opt)
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    n_new = CONTEXT - PROMPT_LEN                 # nobody finishes inside the timed region
    assert warmup + steps + batch + 8 < n_new
    for _ in range(batch):
        eng.add_request([int(t) for t in rng.integers(0, V, PROMPT_LEN)],
                        SamplingParams(max_tokens=n_new, ignore_eos=True))
    while any(r.n_pending > 1 for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()                                           # prefill, and the first token of each
    for _ in range(warmup):
        eng.step()
    torch.cuda.synchronize()
    ctx0 = [r.n_computed for r in eng.scheduler.running]
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(eng.scheduler.running) == batch, "a request finished inside the timed region"
    mean_ctx = sum(ctx0) / batch + steps / 2.0
    for r in list(eng.scheduler.running):
        eng.abort(r.request_id)
    del eng
    torch.cuda.empty_cache()
    return dt, mean_ctx


def run_prefill(model, dtype_name, reps=3, seed=1):
    """Time to first token of one PROMPT_LEN prompt, run as a single step; median of ``reps``."""
    import numpy as np
    import torch
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    opt = EngineOptions(dtype=dtype_name, inflight_slots=1, prefill_chunk_tokens=PROMPT_LEN, page_size=PAGE,
                        ctx_cap=CONTEXT, paged_kv=CONTEXT // PAGE)
    eng = LLMEngine(model, opt)
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    times = []
    for rep in range(reps + 1):
        eng.add_request([int(t) for t in rng.integers(0, V, PROMPT_LEN)], SamplingParams(max_tokens=1, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = eng.step() + eng.flush()          # the first token has reached the host
        torch.cuda.synchronize()
        if rep:
            times.append(time.perf_counter() - t0)
        assert len(done) == 1
    del eng
    torch.cuda.empty_cache()
    return statistics.median(times)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run only the first layers (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--only", choices=["decode", "prefill"], default=None,
                    help="run one part only and print its numbers (for profiling)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2

    import torch
    from flambeau_amd import random_model
    dtype_name = {"bf16": "bfloat16", "fp32": "float32"}[a.dtype]
    el = 2 if a.dtype == "bf16" else 4
    n_layers = a.layers or CONFIG_7B["num_hidden_layers"]
    model, _ = random_model(CONFIG_7B, seed=0, dtype=dtype_name, max_batch_tokens=PROMPT_LEN + 64,
                            std=0.02, gain_std=0.0, n_layers=n_layers)
    sz = sizes(CONFIG_7B, n_layers)

    if a.only == "prefill":
        t = run_prefill(model, dtype_name)
        print(json.dumps({"prefill_ms": round(t * 1e3, 3), "tokens": PROMPT_LEN, "tok_s": round(PROMPT_LEN / t, 1),
                          "frac": round(prefill_flops(sz, PROMPT_LEN) / t / PEAK_FLOPS[a.dtype], 4)}))
        return 0
    if a.only == "decode":
        a.no_points = True

    dt, mean_ctx = run_decode(model, a.batch, a.steps, a.warmup, dtype_name)
    tok_s = a.batch * a.steps / dt
    ms = dt / a.steps * 1e3
    achieved = decode_bytes(sz, a.batch, mean_ctx, el) / (dt / a.steps)
    out = {
        "metric": "decode tok/s (7B, bf16, batch 8, 2,048-token prompts)" if a.dtype == "bf16" and a.batch == 8
        else f"decode tok/s (7B, {a.dtype}, batch {a.batch})",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic: random weights N(0, 0.02^2), uniform random token ids",
        "config": {
            "model": "Mistral-7B-v0.3 sizes", "layers": CONFIG_7B["num_hidden_layers"], "layers_run": n_layers,
            "hidden": 4096, "heads": 32, "kv_heads": 8, "head_dim": 128, "intermediate": 14336, "vocab": 32768,
            "global_batch": a.batch, "seq_len": CONTEXT, "prompt_len": PROMPT_LEN, "page_size": PAGE,
            "sampling": "greedy on device", "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
    }
    if not a.no_points:
        t = run_prefill(model, dtype_name)
        flops = prefill_flops(sz, PROMPT_LEN)
        out["prefill"] = {"value": round(PROMPT_LEN / t, 1), "tokens": PROMPT_LEN, "ms": round(t * 1e3, 3),
                          "frac": round(flops / t / PEAK_FLOPS[a.dtype], 4)}
        points = {}
        for b in (1, 64):
            k = max(16, a.steps // 2)
            dtb, _ = run_decode(model, b, k, min(a.warmup, 8), dtype_name)
            points[f"decode_b{b}"] = round(b * k / dtb, 2)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
