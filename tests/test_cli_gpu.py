"""The command line run as a program on the GPU: ``random-weights`` -> ``inspect`` -> ``infer --json``,
greedy and with seeded temperature draws, with so few slots and pages that requests queue and are
pre-empted; the tokens equal ``generate()``'s and the plain implementation's.  Option names follow
crates/cli/src/main.rs:57-71 (infer) and :124-218 (the serving knobs)."""
import json
import subprocess
import sys

import numpy as np
import pytest

import plain_model as pm
import replay_helpers as rh
from tiny_configs import TINY

pytestmark = pytest.mark.gpu


def _cli(*args):
    r = subprocess.run([sys.executable, "-m", "flambeau_amd", *map(str, args)], capture_output=True, text=True,
                       timeout=600, cwd=str(rh.ROOT))
    assert r.returncode == 0, f"{args}\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    return r


def _plain(d, prompt, n_new, temperature, seed):
    cfg, w = pm.read_model_dir(d)
    rng = pm.Xoshiro(seed)
    toks = list(prompt)
    for _ in range(n_new):
        logits = pm.forward(cfg, w, toks)[-1].astype(np.float32)
        toks.append(pm.sample(logits, rng, temperature=temperature))
    return toks[len(prompt):]


def test_random_weights_inspect_infer(tmp_path):
    t = TINY["B"]
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(t["config"]))
    d = tmp_path / "model"
    _cli("random-weights", "--config", cfg, "--out", d, "--seed", 21, "--std", 0.05, "--gain-std", 0.01, "--dtype", "float32")
    assert "tensors fit the model" in _cli("inspect", d).stdout
    prompts = list(rh.make_requests(384, [3, 30, 17], seed=6).values())
    flags = []
    for p in prompts:
        flags += ["--prompt", ",".join(map(str, p))]
    tight = ["--inflight-slots", 2, "--paged-kv", 5, "--page-size", 16, "--prefill-chunk-tokens", 16, "--max-queue-depth", 4]
    n_new = 18

    # greedy, float32: exactly the plain implementation's tokens, and generate()'s
    out = json.loads(_cli("infer", "--model", d, *flags, "--max-tokens", n_new, "--dtype", "float32", "--json", *tight).stdout)
    assert out["generated"] == 3 * n_new
    for p, o in zip(prompts, out["outputs"]):
        assert o == _plain(d, p, n_new, 0.0, 0)
    from flambeau_amd import generate
    assert generate(str(d), prompts, max_new_tokens=n_new, dtype="float32", inflight_slots=2, paged_kv=5, page_size=16,
                    prefill_chunk_tokens=16) == out["outputs"]

    # seeded temperature draws: request i draws from seed + i
    out_t = json.loads(_cli("infer", "--model", d, *flags, "--max-tokens", n_new, "--dtype", "float32", "--json",
                            "--temperature", 0.8, "--seed", 40, *tight).stdout)
    for i, (p, o) in enumerate(zip(prompts, out_t["outputs"])):
        assert o == _plain(d, p, n_new, 0.8, 40 + i)
    # the host sampler (--no-gpu-sampler) draws the same tokens from the same seeds
    out_h = json.loads(_cli("infer", "--model", d, *flags, "--max-tokens", n_new, "--dtype", "float32", "--json",
                            "--temperature", 0.8, "--seed", 40, "--no-gpu-sampler", *tight).stdout)
    # (both walk the probabilities in index order; their sums differ by rounding alone, which would take a
    # draw within 1e-7 of a boundary to show: none of these 54 is)
    assert out_h["outputs"] == out_t["outputs"]

    # --random-weights CONFIG.json stands for the folder that random-weights writes with that seed
    out_r = json.loads(_cli("infer", "--random-weights", cfg, "--weights-seed", 21, "--weights-std", 0.05,
                            "--weights-gain-std", 0.01, *flags, "--max-tokens", n_new, "--dtype", "float32", "--json", *tight).stdout)
    assert out_r["outputs"] == out["outputs"]

    # text output, bfloat16, a random prompt
    r = _cli("infer", "--model", d, "--random-prompt", 12, "--seed", 3, "--max-tokens", 5, *tight)
    line = r.stdout.strip().splitlines()[0]
    assert line.startswith("[0] ") and len(line.split()) == 6
    assert "5 tokens in" in r.stderr
