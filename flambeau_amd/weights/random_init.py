"""Seeded random weights: as a tensor source, and written out as a model folder.

Matrices and tables are i.i.d. N(0, std^2); norm gains are 1 + N(0, gain_std^2); a part may say
otherwise for a tensor of its own (``TensorSpec.init``: zeros, ones, a bias drawn like a matrix, a
function).  Each tensor
has a generator of its own, seeded from (seed, tensor name), so a tensor's values do not
depend on which others are made.  The reference has no random weights; its tests use a
deterministic signal instead (crates/forward/tests/common/mod.rs:80-86).
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from .safetensors_io import write_safetensors

_TAGS = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16"}


def _tensor_seed(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") & ((1 << 63) - 1)


class RandomSource:
    """A tensor source that makes what the manifest asks for."""

    def __init__(self, manifest: dict, seed: int, std: float = 0.02, gain_std: float = 0.0,
                 store_dtype=torch.bfloat16, device="cpu"):
        self.manifest = manifest
        self.seed = seed
        self.std = std
        self.gain_std = gain_std
        self.store_dtype = store_dtype
        self.device = torch.device(device)
        self.description = f"random weights (seed {seed})"

    def names(self):
        return list(self.manifest)

    def info(self, name):
        tspec = self.manifest[name][2]
        return tuple(tspec.shape), ("I32" if tspec.role == "int32" else _TAGS[self.store_dtype])

    def read(self, name):
        tspec = self.manifest[name][2]
        g = torch.Generator(device=self.device)
        g.manual_seed(_tensor_seed(self.seed, name))
        init = getattr(tspec, "init", None)
        shape = tuple(tspec.shape)
        if callable(init):
            x = init(g, shape, self.device)
            if tuple(x.shape) != shape:
                raise ValueError(f"random weights: the rule of '{name}' made {tuple(x.shape)}, the tensor is {shape}")
            return x.to(torch.int32 if tspec.role == "int32" else self.store_dtype)
        if tspec.role == "int32":
            raise ValueError(f"random weights: no rule for the integer table '{name}' (give its TensorSpec an init function)")
        if init is None:
            init = "gain" if tspec.role == "vector32" else "normal"
        if init == "zeros":
            x = torch.zeros(shape, device=self.device, dtype=torch.float32)
        elif init == "ones":
            x = torch.ones(shape, device=self.device, dtype=torch.float32)
        elif init in ("normal", "gain"):
            x = torch.randn(shape, generator=g, device=self.device, dtype=torch.float32)
            x = 1.0 + x * self.gain_std if init == "gain" else x * self.std
        else:
            raise ValueError(f"random weights: unknown init '{init}' for '{name}'")
        return x.to(self.store_dtype)


def write_random_model(config: dict, out_dir, seed: int, std: float = 0.02, gain_std: float = 0.0,
                       store_dtype=torch.bfloat16):
    """Write ``config.json`` and ``model.safetensors`` for the architecture that
    ``config`` (a config.json dictionary) names.  Returns the folder."""
    from ..models.decoder import DecoderModel
    from ..registry import config_from_dict
    arch, cfg = config_from_dict(config, "config")
    model = DecoderModel(arch.build_spec(cfg), rt=None)
    manifest = model.manifest()
    src = RandomSource(manifest, seed, std, gain_std, store_dtype)
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    cfg_out = dict(config)
    cfg_out["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16",
                              torch.float16: "float16"}[store_dtype]
    (out / "config.json").write_text(json.dumps(cfg_out, indent=2) + "\n")
    items = [(name, tuple(spec[2].shape), torch.int32 if spec[2].role == "int32" else store_dtype, (lambda n=name: src.read(n)))
             for name, spec in manifest.items()]
    write_safetensors(out / "model.safetensors", items,
                      metadata={"format": "pt", "seed": seed, "std": std, "gain_std": gain_std})
    return out
