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
    sys.path.insert(0, str(ROOT))
    import bench
    named = json.loads((ROOT / "BASELINE.json").read_text())["configs"][2]
    c = bench.CONFIG_7B
    for number in (c["num_hidden_layers"], c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                   c["intermediate_size"], c["vocab_size"]):
        assert str(number) in named.replace(",", "")
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
