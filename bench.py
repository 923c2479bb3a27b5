"""Throughput of the engine on one MI355X: decode tokens/s and prefill tokens/s.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 7b|v01-window|24b]

Default run (``--config 7b``): Mistral-7B-v0.3 layer sizes, random weights, bfloat16, a batch of 8
requests that each hold a 2,048-token prompt in the cache and decode greedily (context 2,048 ->
2,304 of 4,096), through the engine's own loop: scheduler, step function, device sampler.  One
"step" is one decode step of the whole batch; K steps are timed three times in a row and the median
is reported.  Prints ONE JSON line; ``value`` is decoded tokens per second.  The same line carries
the 2,048-token prefill, the decode step's memory roofline and decode at batch 1 and 64 (tokens/s,
ms per step and fraction of the roofline each).  Definitions follow the reference's
(doc/PERF_MATRIX.md:5-15): prefill tok/s = prompt tokens / time to first token, decode tok/s over
the decode interval only, median of three repetitions.

``--config v01-window``: Mistral-7B-v0.1 sizes (window 4,096), 8 requests with 8,192-token prompts
run in portions of 512, then 128 decoded tokens each.  ``--config 24b`` and ``--config 12b``: Mistral-Small-24B
and Mistral-Nemo-12B sizes, 64 requests with prompts of 128 to 4,096 tokens and 256 decoded tokens each.  All go through
``LLMEngine`` as a serving loop would drive it and print a line of the same shape.
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

_BASE = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
         "rms_norm_eps": 1e-5, "max_position_embeddings": 32768, "tie_word_embeddings": False}
# Mistral-7B-v0.3 sizes (the benchmark configuration)
CONFIG_7B = dict(_BASE, num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                 head_dim=128, intermediate_size=14336, vocab_size=32768, rope_theta=1e6, sliding_window=None)
# Mistral-7B-v0.1 sizes: a window of 4,096
CONFIG_V01 = dict(CONFIG_7B, vocab_size=32000, rope_theta=10000.0, sliding_window=4096)
# Mistral-Small-24B / Devstral-Small sizes
CONFIG_24B = dict(_BASE, num_hidden_layers=40, hidden_size=5120, num_attention_heads=32, num_key_value_heads=8,
                  head_dim=128, intermediate_size=32768, vocab_size=131072, rope_theta=1e8, sliding_window=None)
# Mistral-Nemo-12B sizes: heads of 128 in a width of 5,120, the 7B feed-forward width, the large vocabulary
CONFIG_12B = dict(_BASE, num_hidden_layers=40, hidden_size=5120, num_attention_heads=32, num_key_value_heads=8,
                  head_dim=128, intermediate_size=14336, vocab_size=131072, rope_theta=1e6, sliding_window=None)
CONFIGS = {"7b": ("Mistral-7B-v0.3 sizes", CONFIG_7B), "v01-window": ("Mistral-7B-v0.1 sizes", CONFIG_V01),
           "24b": ("Mistral-Small-24B sizes", CONFIG_24B), "12b": ("Mistral-Nemo-12B sizes", CONFIG_12B)}
PEAK_HBM = 8.0e12            # bytes/s, MI355X
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PROMPT_LEN = 2048
CONTEXT = 4096
PAGE = 16
REPS = 3


def sizes(cfg, n_layers):
    H, nh, nkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    I, V = cfg["intermediate_size"], cfg["vocab_size"]
    per_layer = (nh + 2 * nkv) * hd * H + H * nh * hd + 3 * I * H
    return dict(matrix_params=n_layers * per_layer, head_params=V * H,
                kv_values_per_token=n_layers * 2 * nkv * hd, nh=nh, hd=hd, n_layers=n_layers)


def decode_bytes(sz, batch, mean_ctx, el):
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    return (sz["matrix_params"] + sz["head_params"]) * el + batch * mean_ctx * sz["kv_values_per_token"] * el


def prefill_flops(sz, T, ctx_before=0, window=0):
    """Flops of a portion of T tokens behind ``ctx_before`` cached ones: products, and attention over
    the keys each query sees (causal, at most ``window``)."""
    gemm = 2.0 * T * sz["matrix_params"] + 2.0 * sz["head_params"]
    keys = 0.0
    for p in (ctx_before, ctx_before + T - 1):            # the mean of first and last query is exact for a linear count
        keys += (min(p + 1, window) if window else p + 1) / 2.0
    attn = sz["n_layers"] * 4.0 * T * keys * sz["hd"] * sz["nh"]
    return gemm + attn


def run_decode(model, batch, steps, warmup, dtype_name, seed=0, reps=REPS):
    """``reps`` times ``steps`` decode steps of ``batch`` requests that each start from a PROMPT_LEN
    prompt in the cache.  Returns per repetition (seconds, mean context length)."""
    import numpy as np
    import torch
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    opt = EngineOptions(dtype=dtype_name, inflight_slots=batch, prefill_chunk_tokens=PROMPT_LEN,
                        page_size=PAGE, ctx_cap=CONTEXT, paged_kv=batch * CONTEXT // PAGE)
    eng = LLMEngine(model, opt)
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    n_new = CONTEXT - PROMPT_LEN                 # nobody finishes inside the timed region
    assert warmup + reps * steps + batch + 8 < n_new, "too many steps for the context"
    for _ in range(batch):
        eng.add_request([int(t) for t in rng.integers(0, V, PROMPT_LEN)],
                        SamplingParams(max_tokens=n_new, ignore_eos=True))
    while any(r.n_pending > 1 for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()                                           # prefill, and the first token of each
    for _ in range(warmup):
        eng.step()
    out = []
    for _ in range(reps):
        torch.cuda.synchronize()
        ctx0 = [r.n_computed for r in eng.scheduler.running]
        t0 = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out.append((dt, sum(ctx0) / batch + steps / 2.0))
    assert len(eng.scheduler.running) == batch, "a request finished inside the timed region"
    for r in list(eng.scheduler.running):
        eng.abort(r.request_id)
    del eng
    torch.cuda.empty_cache()
    return out


def median_rep(reps):
    """The repetition with the median time."""
    return sorted(reps)[len(reps) // 2]


def run_prefill(model, dtype_name, reps=REPS, seed=1):
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


def run_portion(model, dtype_name, portion, ctx_before, reps=REPS, seed=3):
    """Time of one prompt portion of ``portion`` tokens behind ``ctx_before`` cached ones (the context
    is filled in portions of 2,048 first); median of ``reps`` portions that follow one another."""
    import numpy as np
    import torch
    from flambeau_amd.engine import ModelRunner, StepEntry
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    total = ctx_before + (reps + 1) * portion
    runner = ModelRunner(model, n_pages=-(-total // PAGE) + 1, page_size=PAGE, max_slots=1, max_seq_len=total,
                         max_logit_rows=1)
    runner.begin("p")
    ids = lambda n: [int(t) for t in rng.integers(0, V, n)]
    at = 0
    while at < ctx_before:
        k = min(2048, ctx_before - at)
        runner.step([StepEntry("p", ids(k), [])])
        at += k
    times = []
    for rep in range(reps + 1):
        toks = ids(portion)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", toks, [portion - 1])])
        torch.cuda.synchronize()
        if rep:
            times.append(time.perf_counter() - t0)
    runner.end("p")
    del runner
    torch.cuda.empty_cache()
    return statistics.median(times)


def run_decode_filled(model, batch, ctx, steps=24, warmup=6, seed=4):
    """Decode steps of ``batch`` requests that each hold ``ctx`` tokens, without running their prompts:
    the pages are handed out and filled with random values (what attention reads costs the same), then
    single tokens are stepped through ``ModelRunner.step`` (graph replay, no sampling).  Returns
    (seconds per step, mean context)."""
    import numpy as np
    import torch
    from flambeau_amd.engine import ModelRunner, StepEntry
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    total = ctx + steps + warmup + 2
    runner = ModelRunner(model, n_pages=batch * (-(-total // PAGE)) + 2, page_size=PAGE, max_slots=batch, max_seq_len=total,
                         max_logit_rows=batch)
    for pool in runner.storage.pools:
        pool.normal_(0.0, 0.5)
    for i in range(batch):
        runner.begin(i)
        runner.manager.ensure(i, ctx)
        runner.manager.advance(i, ctx)
    step = lambda: runner.step([StepEntry(i, [int(rng.integers(0, V))], [0]) for i in range(batch)])
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    for i in range(batch):
        runner.end(i)
    del runner
    torch.cuda.empty_cache()
    return dt, ctx + warmup + steps / 2.0


def run_enqueue(model, dtype_name, rows=64, decoders=16, seed=2):
    """Host time to enqueue one mixed step of ``rows`` rows (a prompt portion beside ``decoders``
    decoding requests): the time ``ModelRunner.step`` takes to return, the device idle before and
    not waited for after.  Median of the last 30 of 80 steps, in milliseconds (the engine records a
    step's launches and replays them from native code when its shape comes again; shapes that keep
    coming back become graphs)."""
    import numpy as np
    import torch
    from flambeau_amd.engine import ModelRunner, StepEntry
    rng = np.random.default_rng(seed)
    V = model.spec.vocab_size
    runner = ModelRunner(model, n_pages=(decoders + 1) * 4096 // PAGE, page_size=PAGE, max_slots=decoders + 1,
                         max_seq_len=4096, max_logit_rows=decoders + 1)
    ids = lambda n: [int(t) for t in rng.integers(0, V, n)]
    for i in range(decoders):
        runner.begin(i)
    runner.begin("p")
    runner.step([StepEntry(i, ids(60 + 5 * i), []) for i in range(decoders)])
    times = []
    for k in range(80):
        entries = [StepEntry(i, ids(1), [0]) for i in range(decoders)] + [StepEntry("p", ids(rows - decoders), [rows - decoders - 1])]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step(entries)
        times.append(time.perf_counter() - t0)
        torch.cuda.synchronize()
    del runner
    torch.cuda.empty_cache()
    return statistics.median(times[-30:]) * 1e3


def run_serving(model, cfg, dtype_name, prompts, n_new, slots, chunk, ctx):
    """The whole workload through ``LLMEngine`` step by step.  Returns the times of its two phases:
    until the last prompt token has run (portions of prompts beside decoding neighbours), and from
    there on (every step a decode step of the requests still running)."""
    import torch
    from flambeau_amd import EngineOptions, LLMEngine, SamplingParams
    window = cfg["sliding_window"] or 0
    per_req = -(-(min(ctx, window + chunk) if window else ctx) // PAGE) + 2
    opt = EngineOptions(dtype=dtype_name, inflight_slots=slots, prefill_chunk_tokens=chunk, page_size=PAGE,
                        ctx_cap=ctx, paged_kv=slots * per_req, max_batch_tokens=chunk + slots)
    eng = LLMEngine(model, opt)
    reqs = [eng.add_request(p, SamplingParams(max_tokens=n_new, ignore_eos=True)) for p in prompts]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps_a = 0
    while eng.scheduler.waiting or any(r.n_pending > 1 for r in eng.scheduler.running):
        eng.step()
        steps_a += 1
    eng.flush()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    made_a = sum(len(r.output) for r in reqs)
    ctx_a = [r.n_computed for r in eng.scheduler.running]
    steps_b = 0
    while eng.has_work():
        eng.step()
        steps_b += 1
    eng.flush()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    made = sum(len(r.output) for r in reqs)
    assert all(len(r.output) == n_new for r in reqs)
    n_pre = eng.scheduler.n_preemptions
    del eng
    torch.cuda.empty_cache()
    return dict(t_prompt=t1 - t0, t_decode=t2 - t1, steps_prompt=steps_a, steps_decode=steps_b, made_prompt=made_a,
                made_decode=made - made_a, ctx_start=ctx_a, preemptions=n_pre)


def bench_serving(a, name, label, cfg, dtype_name, el):
    import numpy as np
    from flambeau_amd import random_model
    n_layers = a.layers or cfg["num_hidden_layers"]
    rng = np.random.default_rng(5)
    V = cfg["vocab_size"]
    if name == "v01-window":
        batch, n_new, chunk, ctx = 8, 128, 512, 8192 + 128
        lengths = [8192] * batch
        what = "8 requests, 8,192-token prompts in portions of 512, 128 new tokens each"
    else:
        batch, n_new, chunk, ctx = 64, 256, 2048, 4096 + 256
        lengths = [int(n) for n in rng.integers(128, 4097, batch)]
        what = "64 requests, prompts of 128 to 4,096 tokens, 256 new tokens each"
    model, _ = random_model(cfg, seed=0, dtype=dtype_name, max_batch_tokens=chunk + batch, std=0.02, gain_std=0.0,
                            n_layers=n_layers)
    prompts = [[int(t) for t in rng.integers(0, V, n)] for n in lengths]
    sz = sizes(cfg, n_layers)
    runs = [run_serving(model, cfg, dtype_name, prompts, n_new, batch, chunk, ctx) for _ in range(a.reps)]
    r = sorted(runs, key=lambda x: x["t_decode"])[len(runs) // 2]
    window = cfg["sliding_window"] or 0
    extra_points = {}
    if name in ("24b", "12b") and not a.no_points:
        # decode at batch 1 and 8 behind 2,048 tokens each (the cache filled with random values)
        for b in (1, 8):
            dtl, ctxl = run_decode_filled(model, b, PROMPT_LEN, steps=32, warmup=8)
            extra_points[f"decode_b{b}"] = round(b / dtl, 1)
            extra_points[f"decode_b{b}_ms"] = round(dtl * 1e3, 3)
            extra_points[f"decode_b{b}_frac"] = round(decode_bytes(sz, b, ctxl, el) / dtl / PEAK_HBM, 4)
    # the pure decode phase: all requests that are left decode; its bytes from the mean live context
    ms = r["t_decode"] / max(r["steps_decode"], 1) * 1e3
    tok_s = r["made_decode"] / r["t_decode"]
    live = r["made_decode"] / max(r["steps_decode"], 1)                     # mean requests per step
    mean_ctx = (sum(r["ctx_start"]) / max(len(r["ctx_start"]), 1)) + r["steps_decode"] / 2.0
    if window:
        mean_ctx = min(mean_ctx, window)
    achieved = decode_bytes(sz, live, mean_ctx, el) / (ms / 1e3)
    n_prompt = sum(lengths)
    flops = 0.0
    for n in lengths:
        for at in range(0, n, chunk):
            flops += prefill_flops(sz, min(chunk, n - at), at, window)
    out = {
        "metric": f"decode tok/s ({label}, {a.dtype}, {what})",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": r["steps_decode"], "warmup": 0,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic: random weights N(0, 0.02^2), uniform random token ids",
        "config": {
            "model": label, "layers": cfg["num_hidden_layers"], "layers_run": n_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": V, "window": window, "global_batch": batch,
            "seq_len": ctx, "prompt_tokens": n_prompt, "new_tokens": n_new, "portion": chunk, "page_size": PAGE,
            "sampling": "greedy on device", "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
        "prefill": {"value": round(n_prompt / r["t_prompt"], 1), "tokens": n_prompt, "ms": round(r["t_prompt"] * 1e3, 2),
                    "frac": round(flops / r["t_prompt"] / PEAK_FLOPS[a.dtype], 4)},
        "points": {**extra_points, "total_s": round(r["t_prompt"] + r["t_decode"], 3),
                   "overall_generated_tok_s": round(batch * n_new / (r["t_prompt"] + r["t_decode"]), 1),
                   "tokens_decoded_beside_prompts": r["made_prompt"], "mean_live_requests": round(live, 2),
                   "preemptions": r["preemptions"], "reps": a.reps},
    }
    print(json.dumps(out), flush=True)
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=72)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--reps", type=int, default=REPS, help="repetitions of the timed steps; the median is reported")
    ap.add_argument("--config", default="7b", choices=sorted(CONFIGS))
    ap.add_argument("--layers", type=int, default=None, help="run only the first layers (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    ap.add_argument("--only", choices=["decode", "prefill", "enqueue", "portion"], default=None,
                    help="run one part only and print its numbers (for profiling)")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2

    import torch
    from flambeau_amd import random_model
    dtype_name = {"bf16": "bfloat16", "fp32": "float32"}[a.dtype]
    el = 2 if a.dtype == "bf16" else 4
    label, cfg = CONFIGS[a.config]
    if a.config != "7b":
        return bench_serving(a, a.config, label, cfg, dtype_name, el)
    n_layers = a.layers or cfg["num_hidden_layers"]
    model, _ = random_model(cfg, seed=0, dtype=dtype_name, max_batch_tokens=PROMPT_LEN + 64,
                            std=0.02, gain_std=0.0, n_layers=n_layers)
    sz = sizes(cfg, n_layers)

    if a.only == "prefill":
        t = run_prefill(model, dtype_name)
        print(json.dumps({"prefill_ms": round(t * 1e3, 3), "tokens": PROMPT_LEN, "tok_s": round(PROMPT_LEN / t, 1),
                          "frac": round(prefill_flops(sz, PROMPT_LEN) / t / PEAK_FLOPS[a.dtype], 4)}))
        return 0
    if a.only == "enqueue":
        print(json.dumps({"enqueue_ms_mixed64": round(run_enqueue(model, dtype_name), 3)}))
        return 0
    if a.only == "portion":
        t = run_portion(model, dtype_name, 512, 7680)
        print(json.dumps({"portion_ms": round(t * 1e3, 3), "tokens": 512, "context": 7680, "tok_s": round(512 / t, 1)}))
        return 0
    if a.only == "decode":
        a.no_points = True

    # the steps must fit between the prompts' end and the context's: 2,048 -> 2,304 when they fill it
    steps = min(a.steps, (CONTEXT - PROMPT_LEN - a.warmup - a.batch - 9) // a.reps)
    dt, mean_ctx = median_rep(run_decode(model, a.batch, steps, a.warmup, dtype_name, reps=a.reps))
    tok_s = a.batch * steps / dt
    ms = dt / steps * 1e3
    achieved = decode_bytes(sz, a.batch, mean_ctx, el) / (dt / steps)
    out = {
        "metric": "decode tok/s (7B, bf16, batch 8, 2,048-token prompts)" if a.dtype == "bf16" and a.batch == 8
        else f"decode tok/s (7B, {a.dtype}, batch {a.batch})",
        "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic: random weights N(0, 0.02^2), uniform random token ids",
        "config": {
            "model": label, "layers": cfg["num_hidden_layers"], "layers_run": n_layers,
            "hidden": 4096, "heads": 32, "kv_heads": 8, "head_dim": 128, "intermediate": 14336, "vocab": 32768,
            "global_batch": a.batch, "seq_len": CONTEXT, "prompt_len": PROMPT_LEN, "page_size": PAGE,
            "mean_context": round(mean_ctx, 1), "reps": a.reps,
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
            k = min(steps, 40)
            dtb, ctxb = median_rep(run_decode(model, b, k, min(a.warmup, 8), dtype_name, reps=a.reps))
            points[f"decode_b{b}"] = round(b * k / dtb, 2)
            points[f"decode_b{b}_ms"] = round(dtb / k * 1e3, 4)
            points[f"decode_b{b}_frac"] = round(decode_bytes(sz, b, ctxb, el) / (dtb / k) / PEAK_HBM, 4)
        points["enqueue_ms_mixed64"] = round(run_enqueue(model, dtype_name), 3)
        # a portion of 512 tokens behind 8k and 32k of context: tokens/s and the fraction of the matrix peak
        for label, ctx in (("8k", 8192 - 512 * (a.reps + 1)), ("32k", 32768 - 512 * (a.reps + 1))):
            t = run_portion(model, dtype_name, 512, ctx, reps=a.reps)
            mid = ctx + 512 * (a.reps + 1) // 2
            key = f"prefill512_ctx{label}"
            points[key] = round(512 / t, 1)
            points[key + "_frac"] = round(prefill_flops(sz, 512, mid) / t / PEAK_FLOPS[a.dtype], 4)
        # decode behind long contexts (the cache filled with random values, not by running prompts)
        for b, ctx, name in ((8, 16384, "b8_ctx16k"), (8, 32768 - 64, "b8_ctx32k"), (64, 16384, "b64_ctx16k")):
            dtl, ctxl = run_decode_filled(model, b, ctx)
            points[f"decode_{name}"] = round(b / dtl, 1)
            points[f"decode_{name}_ms"] = round(dtl * 1e3, 3)
            points[f"decode_{name}_frac"] = round(decode_bytes(sz, b, ctxl, el) / dtl / PEAK_HBM, 4)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
