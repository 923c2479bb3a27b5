"""Command line: ``python -m flambeau_amd infer|inspect|random-weights``.

Names follow the reference's commands where it has them: ``infer --model --prompt
--max-tokens`` (crates/cli/src/main.rs:57-71), ``inspect`` for its ``inspect-gguf``
(:39,593-625), and the serve knobs ``--inflight-slots``, ``--prefill-chunk-tokens``,
``--paged-kv``, ``--max-queue-depth``, ``--ctx-cap``, ``--no-gpu-sampler`` (:124-218).  There is
no tokenizer here: ``--prompt`` takes token ids separated by commas or blanks, one prompt per
``--prompt``.  ``infer`` and ``inspect`` take ``--random-weights CONFIG.json`` in place of a model
folder: the weights that ``random-weights`` would write for that configuration and seed, without
the folder.
"""
from __future__ import annotations

import argparse
import json
import sys
import time


def _ids(text: str) -> list:
    return [int(t) for t in text.replace(",", " ").split()]


def build_parser():
    ap = argparse.ArgumentParser(prog="flambeau_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)

    inf = sub.add_parser("infer", help="generate from prompts of token ids")
    inf.add_argument("--model", help="folder with config.json and model.safetensors")
    _random_weight_options(inf)
    inf.add_argument("--prompt", action="append", default=[], help="token ids, e.g. '1,5,9'; may repeat")
    inf.add_argument("--random-prompt", type=int, action="append", default=[], metavar="LEN",
                     help="a prompt of LEN uniform random ids (seeded by --seed); may repeat")
    inf.add_argument("--max-tokens", type=int, default=64)
    inf.add_argument("--temperature", type=float, default=0.0)
    inf.add_argument("--top-k", type=int, default=None)
    inf.add_argument("--top-p", type=float, default=None)
    inf.add_argument("--min-p", type=float, default=None)
    inf.add_argument("--repetition-penalty", type=float, default=1.0)
    inf.add_argument("--presence-penalty", type=float, default=0.0)
    inf.add_argument("--frequency-penalty", type=float, default=0.0)
    inf.add_argument("--seed", type=int, default=0)
    inf.add_argument("--ignore-eos", action="store_true")
    inf.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    inf.add_argument("--devices", default="hip:0", help="one device, e.g. hip:0")
    inf.add_argument("--inflight-slots", type=int, default=4)
    inf.add_argument("--prefill-chunk-tokens", type=int, default=512)
    inf.add_argument("--paged-kv", type=int, default=None, metavar="PAGES")
    inf.add_argument("--page-size", type=int, default=16)
    inf.add_argument("--max-queue-depth", type=int, default=16)
    inf.add_argument("--ctx-cap", type=int, default=None)
    inf.add_argument("--no-gpu-sampler", action="store_true")
    inf.add_argument("--json", action="store_true", help="print one JSON object instead of text")

    ins = sub.add_parser("inspect", help="print the configuration and every tensor of a model folder")
    ins.add_argument("path", nargs="?", help="model folder")
    _random_weight_options(ins)

    rnd = sub.add_parser("random-weights", help="write a model folder with seeded random weights")
    rnd.add_argument("--config", required=True, help="a config.json")
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--std", type=float, default=0.02)
    rnd.add_argument("--gain-std", type=float, default=0.0)
    rnd.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    return ap


def _random_weight_options(p) -> None:
    p.add_argument("--random-weights", metavar="CONFIG.json",
                   help="instead of a model folder: seeded random weights for this configuration")
    p.add_argument("--weights-seed", type=int, default=0)
    p.add_argument("--weights-std", type=float, default=0.02)
    p.add_argument("--weights-gain-std", type=float, default=0.0)


def _model_source(a, folder):
    """``("dir", folder)`` or ``("random", config dictionary)``: exactly one of the two must be given."""
    if bool(folder) == bool(a.random_weights):
        raise SystemExit(f"{a.cmd}: give a model folder or --random-weights CONFIG.json (one of the two)")
    if folder:
        return "dir", folder
    with open(a.random_weights) as f:
        return "random", json.load(f)


def _device(devices: str) -> str:
    parts = devices.split(":")
    if parts[0] not in ("hip", "cuda") or (len(parts) > 1 and "," in parts[1]):
        raise SystemExit(f"--devices {devices}: this engine runs on one GPU, e.g. hip:0")
    return f"cuda:{parts[1] if len(parts) > 1 else 0}"


def cmd_infer(a) -> int:
    import numpy as np
    from .engine import EngineOptions, LLMEngine
    from .engine.loading import random_model
    from .registry import config_from_dict, config_from_dir
    from .sampling import SamplingParams
    kind, source = _model_source(a, a.model)
    _, cfg = config_from_dir(source) if kind == "dir" else config_from_dict(source, a.random_weights)
    prompts = [_ids(p) for p in a.prompt]
    rng = np.random.default_rng(a.seed)
    prompts += [[int(t) for t in rng.integers(0, cfg.vocab_size, n)] for n in a.random_prompt]
    if not prompts:
        raise SystemExit("infer: give --prompt or --random-prompt")
    opt = EngineOptions(dtype=a.dtype, device=_device(a.devices), inflight_slots=a.inflight_slots,
                        prefill_chunk_tokens=a.prefill_chunk_tokens, paged_kv=a.paged_kv,
                        page_size=a.page_size, max_queue_depth=a.max_queue_depth, ctx_cap=a.ctx_cap,
                        gpu_sampler=not a.no_gpu_sampler, seed=a.seed)
    if kind == "dir":
        engine = LLMEngine.from_dir(source, opt)
    else:
        # made on the host, tensor by tensor, with the generator that the random-weights command
        # writes folders with: the same seed gives the same model either way
        model, _ = random_model(source, a.weights_seed, dtype=a.dtype, device=opt.device,
                                max_batch_tokens=opt.prefill_chunk_tokens + opt.inflight_slots,
                                std=a.weights_std, gain_std=a.weights_gain_std, generate_on="cpu")
        engine = LLMEngine(model, opt)
    params = [SamplingParams(temperature=a.temperature, top_k=a.top_k, top_p=a.top_p, min_p=a.min_p,
                             repetition_penalty=a.repetition_penalty, presence_penalty=a.presence_penalty,
                             frequency_penalty=a.frequency_penalty, max_tokens=a.max_tokens,
                             seed=a.seed + i, ignore_eos=a.ignore_eos) for i in range(len(prompts))]
    t0 = time.time()
    outs = engine.generate(prompts, params)
    dt = time.time() - t0
    if a.json:
        print(json.dumps({"outputs": outs, "seconds": dt, "generated": sum(map(len, outs))}))
    else:
        for i, o in enumerate(outs):
            print(f"[{i}] " + " ".join(map(str, o)))
        print(f"{sum(map(len, outs))} tokens in {dt:.3f} s", file=sys.stderr)
    return 0


def cmd_inspect(a) -> int:
    from .engine.loading import parse_dtype
    from .models.decoder import DecoderModel
    from .registry import config_from_dict, config_from_dir
    from .weights import RandomSource, SafetensorsDir, check_against_manifest
    kind, source = _model_source(a, a.path)
    arch, cfg = config_from_dir(source) if kind == "dir" else config_from_dict(source, a.random_weights)
    print(f"architecture: {arch.name}")
    for k, v in vars(cfg).items():
        print(f"  {k}: {v}")
    model = DecoderModel(arch.build_spec(cfg), rt=None)
    manifest = model.manifest()
    total = 0
    print("tensors:")
    if kind == "dir":
        src = SafetensorsDir(source)
        for ti in sorted(src.infos(), key=lambda t: t.name):
            print(f"  {ti.name:60s} {ti.dtype:5s} {str(list(ti.shape)):22s} {ti.nbytes:>14,d} B")
            total += ti.numel
    else:
        # what the random-weights command would write: every tensor the model reads, in bfloat16
        src = RandomSource(manifest, a.weights_seed, a.weights_std, a.weights_gain_std, parse_dtype("bfloat16"))
        for name in sorted(manifest):
            shape, tag = src.info(name)
            numel = 1
            for d in shape:
                numel *= d
            print(f"  {name:60s} {tag:5s} {str(list(shape)):22s} {2 * numel:>14,d} B")
            total += numel
    print(f"parameters: {total:,d}")
    specs, shares = model.cache_entries()
    per_token = sum(s.bytes_per_token(1) for s, sh in zip(specs, shares) if s is not None and sh is None)
    print(f"cache per token: {per_token:,d} values ({2 * per_token:,d} B in bfloat16, {4 * per_token:,d} B in float32)")
    skipped = check_against_manifest(manifest, src, model.spec.ignored_tensors)
    print("tensors fit the model" + (f" ({len(skipped)} are not read: {', '.join(skipped)})" if skipped else ""))
    return 0


def cmd_random(a) -> int:
    from .engine.loading import parse_dtype
    from .weights import write_random_model
    with open(a.config) as f:
        config = json.load(f)
    out = write_random_model(config, a.out, a.seed, a.std, a.gain_std, parse_dtype(a.dtype))
    print(out)
    return 0


def main(argv=None) -> int:
    a = build_parser().parse_args(argv)
    return {"infer": cmd_infer, "inspect": cmd_inspect, "random-weights": cmd_random}[a.cmd](a)


if __name__ == "__main__":
    sys.exit(main())
