"""Two further workloads at the layer sizes of real models, two layers each, against the plain
implementation in 32-bit and in bfloat16:

* Mistral-7B-v0.1 sizes with its window of 4,096: a request longer than the window in portions of
  512 beside decoding neighbours, with so few pages that the pages it gives back behind its window
  are handed to a request that starts late.  One key and the queries that look for it are made to
  stand out (a rank-one addition to the first layer's query and key matrices), and the queries sit
  exactly at the window's edge: 4,095 tokens after the key (the last that sees it) and 4,096 after.
* Mistral-Small-24B sizes (width 5120 with 32 heads of 128, so the queries' width differs from the
  model's; feed-forward 32768; vocabulary 131072): whole, last tokens one by one, portions, mixed."""
import math

import numpy as np
import pytest
import torch

import plain_model as pm
import replay_helpers as rh

pytestmark = pytest.mark.gpu

V01 = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
       "num_hidden_layers": 2, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
       "intermediate_size": 14336, "vocab_size": 32000, "rope_theta": 10000.0, "sliding_window": 4096,
       "rms_norm_eps": 1e-5, "max_position_embeddings": 32768, "tie_word_embeddings": False}
SMALL_24B = {"architectures": ["MistralForCausalLM"], "model_type": "mistral", "hidden_act": "silu",
             "num_hidden_layers": 2, "hidden_size": 5120, "num_attention_heads": 32, "num_key_value_heads": 8,
             "head_dim": 128, "intermediate_size": 32768, "vocab_size": 131072, "rope_theta": 1e8,
             "sliding_window": None, "rms_norm_eps": 1e-5, "max_position_embeddings": 32768,
             "tie_word_embeddings": False}

NEEDLE, SEEKER = 17, 23          # the token whose key stands out, and the token whose queries look for it
NEEDLE_AT = 300
WINDOW = 4096


def _write_with_needle(out_dir):
    """Random weights of the 7B-v0.1 sizes; in layer 0 the key of NEEDLE and the queries of SEEKER
    (the four heads of key/value head 0) get a large component along one dim of the slowest rotation
    pair, so that a SEEKER query gives nearly all its weight to a NEEDLE key it can see."""
    from flambeau_amd.weights import SafetensorsFile, write_random_model, write_safetensors
    d = write_random_model(V01, out_dir, seed=31, std=0.02, gain_std=0.01, store_dtype=torch.bfloat16)
    f = SafetensorsFile(d / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    E = t["model.embed_tokens.weight"].double()
    g = t["model.layers.0.input_layernorm.weight"].double()

    def normed(tok):
        x = E[tok]
        return x / torch.sqrt((x * x).mean() + 1e-5) * g

    hd, beta, dim = 128, 13.0, 63                   # dim 63 pairs with 127: the pair that turns slowest
    nb, nc = normed(NEEDLE), normed(SEEKER)
    wk = t["model.layers.0.self_attn.k_proj.weight"].double()
    wk[dim] += beta * nb / (nb @ nb)
    t["model.layers.0.self_attn.k_proj.weight"] = wk.to(torch.bfloat16)
    wq = t["model.layers.0.self_attn.q_proj.weight"].double()
    for head in range(4):
        wq[head * hd + dim] += beta * nc / (nc @ nc)
    t["model.layers.0.self_attn.q_proj.weight"] = wq.to(torch.bfloat16)
    write_safetensors(d / "model.safetensors", t)
    return d


@pytest.fixture(scope="module")
def window_case(tmp_path_factory):
    d = _write_with_needle(tmp_path_factory.mktemp("v01") / "model")
    rng = np.random.default_rng(77)

    def ids(n):
        t = rng.integers(30, 32000, n)             # never NEEDLE or SEEKER by chance
        return [int(x) for x in t]

    long = ids(4700)
    long[NEEDLE_AT] = NEEDLE
    for p in (NEEDLE_AT + 100, NEEDLE_AT + WINDOW - 1, NEEDLE_AT + WINDOW, 4650):
        long[p] = SEEKER
    reqs = {"long": long, "n1": ids(640), "n2": ids(700), "late": ids(400)}
    # wanted places: the ends of the long request's portions, a run of places across the window's
    # edge, and everything the neighbours decode
    edge = list(range(NEEDLE_AT + WINDOW - 3, NEEDLE_AT + WINDOW + 3))
    cfg, w = pm.read_model_dir(d)
    ref = {}
    long_rows = sorted(set(list(range(511, 4700, 512)) + edge + [NEEDLE_AT + 100, 4650, 4699, 0, 1]))
    ref["long"] = dict(zip(long_rows, pm.forward(cfg, w, long, rows=long_rows)))
    for rid in ("n1", "n2", "late"):
        toks = reqs[rid]
        rows = list(range(len(toks) - 60, len(toks))) if rid != "late" else [0, 199, 399]
        ref[rid] = dict(zip(rows, pm.forward(cfg, w, toks, rows=rows)))
    # The case is sensitive to the window's edge: with a window one key longer the query just past the
    # edge would still see NEEDLE, with a window one key shorter the query at the edge would not.
    upto = NEEDLE_AT + WINDOW + 1
    longer = pm.forward(dict(cfg, sliding_window=WINDOW + 1), w, long[:upto], rows=[NEEDLE_AT + WINDOW])[0]
    shorter = pm.forward(dict(cfg, sliding_window=WINDOW - 1), w, long[:upto], rows=[NEEDLE_AT + WINDOW - 1])[0]
    sensitivity = min(float(np.abs(longer - ref["long"][NEEDLE_AT + WINDOW]).max()),
                      float(np.abs(shorter - ref["long"][NEEDLE_AT + WINDOW - 1]).max()))
    return d, reqs, ref, sensitivity


def _steps(reqs, ref):
    """The long request in portions of 512; n1 and n2 have their prompts run first and then decode one
    token per step beside it; 'late' starts when the long request has passed its window."""
    steps = []
    want_of = {rid: set(r) for rid, r in ref.items()}

    def entry(rid, a, b):
        return dict(id=rid, tokens=reqs[rid][a:b], want=[p - a for p in sorted(want_of[rid]) if a <= p < b])

    steps.append(dict(entries=[entry("n1", 0, 580), entry("n2", 0, 640)], end=[]))
    at = {"long": 0, "n1": 580, "n2": 640, "late": 0}
    while at["long"] < len(reqs["long"]):
        entries = []
        k = min(512, len(reqs["long"]) - at["long"])
        entries.append(entry("long", at["long"], at["long"] + k))
        at["long"] += k
        for rid in ("n1", "n2"):
            for _ in range(1):
                if at[rid] < len(reqs[rid]) - 4:
                    entries.append(entry(rid, at[rid], at[rid] + 1))
                    at[rid] += 1
        if at["long"] > WINDOW + 512 and at["late"] < len(reqs["late"]):
            k = min(200, len(reqs["late"]) - at["late"])
            entries.append(entry("late", at["late"], at["late"] + k))
            at["late"] += k
        steps.append(dict(entries=entries, end=[]))
    # the neighbours' remaining tokens one by one, then everybody ends
    while any(at[r] < len(reqs[r]) for r in ("n1", "n2", "late")):
        entries = []
        for rid in ("n1", "n2", "late"):
            if at[rid] < len(reqs[rid]):
                k = 1 if rid != "late" else min(200, len(reqs[rid]) - at[rid])
                entries.append(entry(rid, at[rid], at[rid] + k))
                at[rid] += k
        steps.append(dict(entries=entries, end=[]))
    steps[-1]["end"] = list(reqs)
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_of_4096_at_real_layer_sizes(window_case, dtype):
    from flambeau_amd.engine import ModelRunner, load_model
    d, reqs, ref, sensitivity = window_case
    scale = max(float(np.abs(r).max()) for rr in ref.values() for r in rr.values())
    # a window off by one key in either direction moves the logits at the edge by far more than the tolerance
    assert sensitivity > 5 * rh.tolerance("bfloat16", scale), sensitivity
    model, _ = load_model(d, dtype=dtype, max_batch_tokens=1280)
    # pages: the long request's window and one portion, the two neighbours, and not enough for 'late'
    # until the long request has given pages back
    ps = 16
    n_pages = (WINDOW + 512) // ps + 1 + 41 + 45 + 12
    runner = ModelRunner(model, n_pages=n_pages, page_size=ps, max_slots=4, max_logit_rows=1280)
    runner.storage.fill(float("nan"))
    steps = _steps(reqs, ref)
    got = rh.run_in_process(runner, steps)
    pool = runner.manager.pools[0]
    assert not runner.manager.live and pool.n_free == pool.n_pages
    total = sum(-(-len(t) // ps) for t in reqs.values())
    assert pool.n_acquired == total > pool.n_pages              # pages were given back mid-request and used again
    tol = rh.tolerance(dtype, scale)
    worst = 0.0
    for (rid, p), row in sorted(got.items()):
        diff = float(np.abs(row - ref[rid][p]).max())
        worst = max(worst, diff)
        assert diff <= tol, f"{dtype}: request {rid} position {p} differs by {diff:.3g} (tolerance {tol:.3g})"
    assert len(got) == sum(len(r) for r in ref.values())
    print(f"window 4096 at 7B layer sizes [{dtype}]: worst difference {worst:.3g} at logits up to {scale:.3g}")


@pytest.fixture(scope="module")
def small24b_dir(tmp_path_factory):
    from flambeau_amd.weights import write_random_model
    return write_random_model(SMALL_24B, tmp_path_factory.mktemp("s24b") / "model", seed=13, std=0.02, gain_std=0.01,
                              store_dtype=torch.bfloat16)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cutting_at_24b_layer_sizes(small24b_dir, dtype):
    from flambeau_amd.engine import ModelRunner, load_model
    reqs = rh.make_requests(131072, [130, 37, 75], seed=19)
    ref = rh.plain_logits(small24b_dir, reqs)
    model, _ = load_model(small24b_dir, dtype=dtype, max_batch_tokens=256)
    runner = ModelRunner(model, n_pages=20, page_size=16, max_slots=4, max_logit_rows=256)
    runner.storage.fill(float("nan"))
    for what, steps in (("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs, tail=20)),
                        ("portions", rh.trace_portions(reqs, sizes=(2, 66, 3, 17, 40, 5))),
                        ("mixed", rh.trace_mixed(reqs, seed=3, max_portion=70))):
        got = rh.run_in_process(runner, steps)
        assert not runner.manager.live
        worst = rh.compare(got, reqs, ref, dtype, f"24B sizes {what}")
    print(f"24B layer sizes [{dtype}]: worst difference in the mixed cutting {worst:.3g}")
