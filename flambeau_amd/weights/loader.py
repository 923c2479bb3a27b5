"""Loading a model's tensors by name.

A ``TensorSource`` hands out host tensors by name: a model folder with
``model.safetensors`` (or shards listed in ``model.safetensors.index.json``), or the
seeded random generator.  ``load_weights`` compares what the model asks for with what the
source holds and raises ONE error that lists every missing tensor, every unexpected one and
every wrong shape; then it moves the tensors to the device one by one, matrices and tables
in the compute dtype, norm gains in float32 (a tensor stored in 32-bit keeps its precision
when its role allows it), integer tables as int32.

Reference: tensors by name with an error for an unknown one
(crates/quant/src/gguf.rs:370-373, crates/quant/src/error.rs:27-28); element-count check per
tensor (crates/forward/src/loader/primitives.rs:158-163).
"""
from __future__ import annotations

import fnmatch
import json
import warnings
from pathlib import Path

import torch

from .safetensors_io import SafetensorsFile, WeightFileError


class WeightError(ValueError):
    """The tensors of a source do not fit the model.  ``missing``, ``unexpected`` and
    ``wrong_shape`` hold the details that the message lists."""

    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = [f"{where}: the tensors do not fit the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, got, want in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, expected {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is {got}, expected a float type (F32, BF16, F16)")
        super().__init__("\n".join(lines))


_FLOAT_TAGS = ("F32", "BF16", "F16", "F64")
_INT_TAGS = ("I32", "I64", "I16", "I8", "U8")


class SafetensorsDir:
    """The tensors of a model folder."""

    def __init__(self, model_dir):
        self.dir = Path(model_dir)
        index = self.dir / "model.safetensors.index.json"
        single = self.dir / "model.safetensors"
        self._files: dict[str, SafetensorsFile] = {}
        self._where: dict[str, str] = {}
        if single.is_file():
            f = SafetensorsFile(single)
            self._files[single.name] = f
            for n in f.names():
                self._where[n] = single.name
        elif index.is_file():
            weight_map = json.loads(index.read_text()).get("weight_map")
            if not isinstance(weight_map, dict):
                raise WeightFileError(f"{index}: no 'weight_map'")
            for shard in sorted(set(weight_map.values())):
                self._files[shard] = SafetensorsFile(self.dir / shard)
            for n, shard in weight_map.items():
                if n not in self._files[shard].tensors:
                    raise WeightFileError(f"{index}: tensor '{n}' is not in {shard}")
                self._where[n] = shard
        else:
            raise WeightFileError(f"{self.dir}: neither model.safetensors nor model.safetensors.index.json")
        self.description = str(self.dir)

    def names(self):
        return list(self._where)

    def info(self, name):
        ti = self._files[self._where[name]].info(name)
        return ti.shape, ti.dtype

    def read(self, name):
        return self._files[self._where[name]].read(name)

    def infos(self):
        return [self._files[self._where[n]].info(n) for n in self._where]

    def close(self):
        for f in self._files.values():
            f.close()


def check_against_manifest(manifest: dict, source, ignored=()) -> list:
    """Raises ONE ``WeightError`` for everything that does not fit.  ``ignored``: name patterns
    (``fnmatch``) of tensors the architecture says a file may hold without the model reading them;
    those are skipped with a warning and returned."""
    have = set(source.names())
    want = set(manifest)
    missing = want - have
    unexpected = have - want
    skipped = sorted(n for n in unexpected if any(fnmatch.fnmatchcase(n, pat) for pat in ignored))
    unexpected -= set(skipped)
    if skipped:
        warnings.warn(f"{source.description}: {len(skipped)} tensors are not read by this model: "
                      + ", ".join(skipped[:8]) + (" ..." if len(skipped) > 8 else ""), stacklevel=2)
    wrong_shape, wrong_dtype = [], []
    for name in want & have:
        shape, tag = source.info(name)
        tspec = manifest[name][2]
        if tuple(shape) != tuple(tspec.shape):
            wrong_shape.append((name, tuple(shape), tuple(tspec.shape)))
        ok = _INT_TAGS if tspec.role == "int32" else _FLOAT_TAGS
        if tag not in ok:
            wrong_dtype.append((name, tag))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(source.description, missing, unexpected, wrong_shape, wrong_dtype)
    return skipped


def load_weights(model, source, progress=None) -> None:
    """Check, move to the device, bind."""
    manifest = model.manifest()
    check_against_manifest(manifest, source, getattr(model.spec, "ignored_tensors", ()))
    tensors = {}
    for i, (name, (_, _, tspec)) in enumerate(manifest.items()):
        tensors[name] = model.rt.to_device(source.read(name), tspec.role)
        if progress is not None:
            progress(i + 1, len(manifest), name)
    model.bind(tensors)
