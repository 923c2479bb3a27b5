"""Trace replay over the engine's step function (the program behind ``bin/trace_run``).

It samples nothing and has no forward pass, cache or loader of its own: requests are begun
and ended on the ``ModelRunner`` that generation uses, and every step is one call of its
``step``.  The reference's counterpart feeds a fixed id list one token per step and appends
the logits to a file (crates/models/qwen35-v2/tests/parity_dump_v2.rs:41-50).
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path

PAGE_ROUNDING = 64   # live requests' token counts are rounded up to this when sizing the pool


def build_parser():
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (divides 64)")
    ap.add_argument("--max-slots", type=int, default=64, help="most requests live at a time")
    ap.add_argument("--plain-kernels", action="store_true",
                    help="run the plain kernels in bfloat16 too (float32 always does)")
    ap.add_argument("--poison-cache", action="store_true",
                    help="fill the cache with NaN before the first step: a read of a row that was never "
                         "written then shows in the logits")
    return ap


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    if args.page_size < 1 or PAGE_ROUNDING % args.page_size:
        print(f"trace_run: --page-size must divide {PAGE_ROUNDING}", file=sys.stderr)
        return 2
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)

    import numpy as np
    import torch
    from .engine import ModelRunner, StepEntry, load_model

    max_tokens = max(PAGE_ROUNDING, -(-args.max_tokens // PAGE_ROUNDING) * PAGE_ROUNDING)
    model, _ = load_model(args.model, dtype=args.dtype, max_batch_tokens=max_tokens,
                          tuned=not args.plain_kernels)
    runner = ModelRunner(model, n_pages=max_tokens // args.page_size, page_size=args.page_size,
                         max_slots=args.max_slots, max_logit_rows=max_tokens)
    if args.poison_cache:
        runner.storage.fill(float("nan"))

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step_no = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if rid not in runner.manager.live and not runner.begin(rid):
                raise RuntimeError(f"step {step_no}: no free slot for request {rid!r}")
            entries.append(StepEntry(rid, list(e["tokens"]), list(e.get("want", []))))
        logits = runner.step(entries) if entries else None
        if logits is not None and logits.shape[0] > 0:
            arr = logits.to("cpu", torch.float32).numpy().astype("<f4", copy=False)
            tmp = out_dir / f".{step_no}.f32.tmp"
            arr.tofile(tmp)
            tmp.replace(out_dir / f"{step_no}.f32")
        else:
            torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if rid in runner.manager.live:
                runner.end(rid)
        print(f"done {step_no}", flush=True)
    pools = runner.manager.pools
    print(f"trace_run: {sum(p.n_pages for p in pools)} pages in the pool, {sum(p.n_acquired for p in pools)} handed out",
          file=sys.stderr)
    return 0
