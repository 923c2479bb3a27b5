"""Traces for the tests: the same requests cut into steps in different ways, run through the
engine's step function (in process) or through bin/trace_run (as a program), and compared
with the plain implementation position by position."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np

import plain_model as pm

ROOT = Path(__file__).resolve().parent.parent


def make_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, vocab, n)] for i, n in enumerate(lengths)}


# ------------------------------------------------------------------ ways of cutting
def trace_whole(requests):
    """Each request alone and whole, every position wanted."""
    return [dict(entries=[dict(id=rid, tokens=toks, want=list(range(len(toks))))], end=[rid])
            for rid, toks in requests.items()]


def trace_tail(requests, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append(dict(entries=[dict(id=rid, tokens=toks[:head], want=list(range(head)))], end=[]))
        for i in range(head, len(toks)):
            steps.append(dict(entries=[dict(id=rid, tokens=[toks[i]], want=[0])], end=[]))
        steps[-1]["end"] = [rid]
    return steps


def trace_portions(requests, sizes=(2, 5, 3, 17, 2, 8, 31, 4, 2, 64, 9)):
    """Portions of changing size, down to two tokens (a last single token if it must be)."""
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            steps.append(dict(entries=[dict(id=rid, tokens=toks[at:at + n], want=list(range(n)))], end=[]))
            at += n
            k += 1
        steps[-1]["end"] = [rid]
    return steps


def trace_mixed(requests, seed, max_live=4, decode_tail=12, max_portion=24, idle_prob=0.15):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of others;
    requests sometimes sit a step out; a finished request makes room for the next, whose pages
    are the ones just given back."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live = {}          # rid -> position
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            toks = requests[rid]
            at = live[rid]
            if len(live) > 1 and rng.random() < idle_prob:
                continue
            left = len(toks) - at
            if left <= decode_tail:
                n = 1
            else:
                n = int(min(left - decode_tail, rng.integers(2, max_portion + 1)))
            # wanted places: all of a short portion, both ends of a long one, sometimes none
            if n <= 4:
                want = list(range(n))
            elif rng.random() < 0.2:
                want = []
            else:
                want = sorted({0, n // 2, n - 1})
            entries.append(dict(id=rid, tokens=toks[at:at + n], want=want))
            live[rid] = at + n
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            order = rng.permutation(len(entries))
            steps.append(dict(entries=[entries[i] for i in order], end=end))
    return steps


def peak_tokens(steps, rounding=64):
    """Most tokens live requests hold at any time, each request's count rounded up."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-v // rounding) * rounding for v in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


# ------------------------------------------------------------------ running a trace
def run_in_process(runner, steps):
    """``{(request, position): logits}`` through ``ModelRunner.step``."""
    from flambeau_amd.engine import StepEntry
    out, pos = {}, {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in runner.manager.live:
                assert runner.begin(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = runner.step(entries)
        rows = logits.cpu().double().numpy() if logits is not None else None
        k = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = rows[k]
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
        for rid in s["end"]:
            runner.end(rid)
        runner.manager.check_invariants()
    return out


def run_program(model_dir, dtype, steps, out_dir, max_tokens, vocab, extra=(), timeout=600, stats=None):
    """The same through ``bin/trace_run`` as a child process.  ``stats`` (a dict) receives the pool's
    size and the number of pages handed out, which the program reports when its input ends."""
    lines = "".join(json.dumps(dict(step=i, **s)) + "\n" for i, s in enumerate(steps))
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens), *extra]
    r = subprocess.run(cmd, input=lines, capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, f"trace_run failed ({r.returncode}):\n{r.stdout[-2000:]}\n{r.stderr[-4000:]}"
    done = [l for l in r.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(steps))], r.stdout[-2000:]
    if stats is not None:
        import re
        m = re.search(r"trace_run: (\d+) pages in the pool, (\d+) handed out", r.stderr)
        assert m, r.stderr[-2000:]
        stats["pool"], stats["handed_out"] = int(m.group(1)), int(m.group(2))
    out, pos = {}, {}
    for i, s in enumerate(steps):
        n_want = sum(len(e["want"]) for e in s["entries"])
        f = Path(out_dir) / f"{i}.f32"
        if n_want == 0:
            assert not f.exists()
        else:
            rows = np.fromfile(f, dtype="<f4").reshape(n_want, vocab).astype(np.float64)
        k = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                out[(e["id"], base + w)] = rows[k]
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
    return out


# ------------------------------------------------------------------ comparing
_plain_cache = {}


def plain_logits(model_dir, requests):
    """Plain logits of every request, whole; cached per (folder, tokens)."""
    out = {}
    cfg = w = None
    for rid, toks in requests.items():
        key = (str(model_dir), tuple(toks))
        if key not in _plain_cache:
            if cfg is None:
                cfg, w = pm.read_model_dir(model_dir)
            _plain_cache[key] = pm.forward(cfg, w, toks)
        out[rid] = _plain_cache[key]
    return out


def tolerance(dtype, ref_scale):
    """float32: 1e-4 absolute.  bfloat16: activations between kernels carry 8 significant bits
    (relative step 2^-8), so after a few layers the logits are off by some 1e-3 of their scale;
    2e-2 of the largest logit bounds that with room and is far below what a wrong key, a wrong
    position or a stale page does (tens of percent)."""
    return 1e-4 if dtype == "float32" else 2e-2 * ref_scale


def compare(got, requests, ref, dtype, what):
    worst = 0.0
    scale = max(float(np.abs(r).max()) for r in ref.values())
    tol = tolerance(dtype, scale)
    bad = []
    for (rid, p), row in sorted(got.items()):
        d = float(np.abs(row - ref[rid][p]).max())
        worst = max(worst, d)
        if not d <= tol:
            bad.append((rid, p, d))
    assert not bad, (f"{what} [{dtype}]: {len(bad)} of {len(got)} positions differ by more than {tol:.3g}; "
                     f"first wrong: request {bad[0][0]} position {bad[0][1]} (diff {bad[0][2]:.3g})")
    return worst
