"""What can be said about the entry points without a GPU: bench.py refuses more than one GPU, its
sizes are the named configuration's, the command line knows the reference's option names."""
import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bench_runs_the_named_configuration():
    """The default run has the sizes of Mistral-7B-v0.3: 32 layers, width 4096, 32 heads in 8 groups of
    128, feed-forward 14336, vocabulary 32768, theta 1e6, no window; prompts of 2,048 tokens in a
    context of 4,096, pages of 16."""
    sys.path.insert(0, str(ROOT))
    import bench
    c = bench.CONFIG_7B
    assert (c["num_hidden_layers"], c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"],
            c["intermediate_size"], c["vocab_size"], c["rope_theta"], c["sliding_window"]) == \
        (32, 4096, 32, 8, 128, 14336, 32768, 1e6, None)
    assert bench.CONTEXT == 4096 and bench.PROMPT_LEN == 2048 and bench.PAGE == 16


def test_command_line_has_the_reference_option_names():
    r = subprocess.run([sys.executable, "-m", "flambeau_amd", "infer", "--help"], capture_output=True, text=True,
                       timeout=120, cwd=str(ROOT))
    assert r.returncode == 0
    # crates/cli/src/main.rs:124-218 (serve flags), runtime/src/sampling.rs:39-50 (sampling options)
    for option in ("--inflight-slots", "--prefill-chunk-tokens", "--paged-kv", "--max-queue-depth", "--ctx-cap",
                   "--no-gpu-sampler", "--temperature", "--top-k", "--top-p", "--min-p", "--repetition-penalty",
                   "--presence-penalty", "--frequency-penalty", "--seed", "--max-tokens"):
        assert option in r.stdout, option


def _cli(*args, cwd=None):
    r = subprocess.run([sys.executable, "-m", "flambeau_amd", *args], capture_output=True, text=True, timeout=300,
                       cwd=str(ROOT))
    return r


def test_random_weights_and_inspect_run_without_a_gpu(tmp_path):
    """``random-weights`` writes a folder, ``inspect`` reads it back and checks it against the model;
    ``inspect --random-weights`` lists the same tensors without a folder (crates/cli/src/main.rs:593-625
    lists tensors, types and metadata of a file in the same manner)."""
    sys.path.insert(0, str(ROOT / "tests"))
    from tiny_configs import TINY
    cfg = tmp_path / "tiny.json"
    cfg.write_text(json.dumps(TINY["B"]["config"]))
    out = tmp_path / "model"
    r = _cli("random-weights", "--config", str(cfg), "--out", str(out), "--seed", "3", "--std", "0.05", "--dtype", "float32")
    assert r.returncode == 0, r.stderr[-2000:]
    assert (out / "config.json").is_file() and (out / "model.safetensors").is_file()
    r = _cli("inspect", str(out))
    assert r.returncode == 0, r.stderr[-2000:]
    for piece in ("architecture: MistralForCausalLM", "num_key_value_heads: 1", "head_dim: 24", "rope_theta: 1000000.0",
                  "model.layers.2.mlp.down_proj.weight", "[96, 224]", "F32", "tensors fit the model", "cache per token: 144 values"):
        assert piece in r.stdout, piece
    n_params = 2 * 384 * 96 + 3 * (96 * 144 + 2 * 24 * 96 + 144 * 96 + 3 * 96 * 224 + 2 * 96) + 96
    assert f"parameters: {n_params:,d}" in r.stdout
    r2 = _cli("inspect", "--random-weights", str(cfg))
    assert r2.returncode == 0, r2.stderr[-2000:]
    assert f"parameters: {n_params:,d}" in r2.stdout and "BF16" in r2.stdout and "tensors fit the model" in r2.stdout
    names = lambda text: sorted(l.split()[0] for l in text.splitlines() if l.startswith("  model.") or l.startswith("  lm_head"))
    assert names(r.stdout) == names(r2.stdout) and len(names(r.stdout)) == 3 * 9 + 3
    # a folder and --random-weights together, or neither, is refused
    assert _cli("inspect").returncode != 0
    assert _cli("inspect", str(out), "--random-weights", str(cfg)).returncode != 0
    # a tensor too many in the file is named
    import torch
    from flambeau_amd.weights import SafetensorsFile, write_safetensors
    f = SafetensorsFile(out / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(12)
    write_safetensors(out / "model.safetensors", t)
    r = _cli("inspect", str(out))
    assert r.returncode == 0 and "1 are not read: model.layers.0.self_attn.rotary_emb.inv_freq" in r.stdout
    t["extra.weight"] = torch.zeros(3)
    write_safetensors(out / "model.safetensors", t)
    r = _cli("inspect", str(out))
    assert r.returncode != 0 and "unexpected (1): extra.weight" in r.stderr
