"""From a model folder (or a configuration and a seed) to a model on the device."""
from __future__ import annotations

import torch

from ..models.decoder import DecoderModel
from ..registry import config_from_dict, config_from_dir
from ..weights.loader import SafetensorsDir, load_weights
from ..weights.random_init import RandomSource
from .runtime import Runtime

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {name!r}") from None


def load_model(model_dir, dtype="bfloat16", device="cuda:0", max_batch_tokens: int = 2048, tuned: bool = True):
    """The model of ``model_dir`` (class chosen by its config.json), weights on the device."""
    arch, cfg = config_from_dir(model_dir)
    rt = Runtime(device, parse_dtype(dtype), max_batch_tokens, tuned)
    model = DecoderModel(arch.build_spec(cfg), rt)
    src = SafetensorsDir(model_dir)
    try:
        load_weights(model, src)
    finally:
        src.close()
    return model, cfg


def random_model(config: dict, seed: int, dtype="bfloat16", device="cuda:0", max_batch_tokens: int = 2048,
                 tuned: bool = True, std: float = 0.02, gain_std: float = 0.0, n_layers: int | None = None,
                 generate_on: str = "device"):
    """A model with seeded random weights, without a folder.  ``n_layers`` keeps only the first layers
    of the configuration (for measurements that say so).  ``generate_on``: "device" makes the
    tensors with the GPU's generator (fast; its values are its own), "cpu" with the host's, which
    gives the values that ``write_random_model`` writes for the same seed."""
    arch, cfg = config_from_dict(config, "config")
    rt = Runtime(device, parse_dtype(dtype), max_batch_tokens, tuned)
    spec = arch.build_spec(cfg)
    if n_layers is not None and n_layers < len(spec.layers):
        spec.layers = spec.layers[:n_layers]
        spec.run_order = [e for e in spec.run_order if e.layer < n_layers]
    model = DecoderModel(spec, rt)
    if generate_on not in ("device", "cpu"):
        raise ValueError(f"generate_on must be 'device' or 'cpu', got {generate_on!r}")
    src = RandomSource(model.manifest(), seed, std, gain_std, rt.dtype,
                       device=rt.device if generate_on == "device" else "cpu")
    load_weights(model, src)
    return model, cfg
