"""bin/trace_run as a program: the same requests whole, with the last 32 tokens one by one, in
portions of changing size, and mixed with so few pages that they are used again; in 32-bit and
in bfloat16; all compared with the plain implementation."""
import json
import subprocess
import sys

import numpy as np
import pytest

import replay_helpers as rh
from tiny_configs import TINY

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_in_all_cuttings(model_dirs, tmp_path, name, dtype):
    """The cache starts full of NaN, so a read of a row that was never written shows; the mixed trace
    holds so many requests that the pool (sized, as the program's contract says, for the most
    tokens live at a time, each request rounded up to 64) hands its pages out several times."""
    d = model_dirs[(name, dtype)]
    vocab = TINY[name]["config"]["vocab_size"]
    lengths = {"A": [40, 70, 97, 33, 64, 12, 90, 55, 128, 21, 77, 64, 100, 38],
               "B": [97, 1, 150, 64, 31, 33, 120, 200, 17, 65, 180, 96, 2, 140]}[name]
    reqs = rh.make_requests(vocab, lengths, seed=5)
    ref = rh.plain_logits(d, reqs)
    for mode, steps in [("whole", rh.trace_whole(reqs)), ("tail", rh.trace_tail(reqs)),
                        ("portions", rh.trace_portions(reqs)), ("mixed", rh.trace_mixed(reqs, seed=13))]:
        out = tmp_path / mode
        stats = {}
        got = rh.run_program(d, dtype, steps, out, rh.peak_tokens(steps), vocab, extra=("--poison-cache",), stats=stats)
        assert got, mode
        # pages were used again, in every mode (one process and one pool per mode)
        assert 2 * stats["handed_out"] > 3 * stats["pool"], (mode, stats)
        rh.compare(got, reqs, ref, dtype, f"trace_run {name} {mode}")


def test_replay_details(model_dirs, tmp_path):
    """A request may sit out a step; a step may want nothing (no file) or hold no entries; files
    are little-endian float32 [wanted, vocab] in the order of entries and of want."""
    d = model_dirs[("A", "float32")]
    reqs = rh.make_requests(256, [10, 6, 2], seed=8)
    a, b, c = reqs["r0"], reqs["r1"], reqs["r2"]
    steps = [
        dict(entries=[dict(id="r0", tokens=a[:4], want=[])], end=[]),
        dict(entries=[dict(id="r1", tokens=b[:3], want=[2, 0])], end=[]),
        dict(entries=[], end=[]),
        dict(entries=[dict(id="r1", tokens=b[3:], want=[2]), dict(id="r0", tokens=a[4:], want=[5, 0])], end=["r0", "r1"]),
        # every token of the step wanted, out of order; then one place twice
        dict(entries=[dict(id="r2", tokens=c, want=[1, 0])], end=["r2"]),
        dict(entries=[dict(id="r2", tokens=c, want=[0, 0])], end=["r2"]),
    ]
    lines = "".join(json.dumps(dict(step=10 + i, **s)) + "\n" for i, s in enumerate(steps))
    out = tmp_path / "o"
    r = subprocess.run([sys.executable, str(rh.ROOT / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128"], input=lines, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    assert r.stdout.split() == ["done", "10", "done", "11", "done", "12", "done", "13", "done", "14", "done", "15"]
    assert sorted(p.name for p in out.iterdir()) == ["11.f32", "13.f32", "14.f32", "15.f32"]
    ref = rh.plain_logits(d, reqs)
    s11 = np.fromfile(out / "11.f32", dtype="<f4").reshape(2, 256)
    s13 = np.fromfile(out / "13.f32", dtype="<f4").reshape(3, 256)
    s14 = np.fromfile(out / "14.f32", dtype="<f4").reshape(2, 256)
    s15 = np.fromfile(out / "15.f32", dtype="<f4").reshape(2, 256)
    assert np.abs(ref["r2"][0] - ref["r2"][1]).max() > 1e-3          # the two rows can be told apart
    for row, (rid, p) in zip(list(s11) + list(s13) + list(s14) + list(s15),
                             [("r1", 2), ("r1", 0), ("r1", 5), ("r0", 9), ("r0", 4), ("r2", 1), ("r2", 0), ("r2", 0), ("r2", 0)]):
        assert np.abs(row - ref[rid][p]).max() < 1e-4
