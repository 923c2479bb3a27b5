"""Reading and writing safetensors files by tensor name.

File format: 8 bytes little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets}}``, then the data.  Tensors are memory
mapped and handed out one by one, so a large file never sits in host memory as a
whole.  Counterpart of the reference's by-name access to its own input format
(crates/quant/src/gguf.rs:370-373 ``info``, :466-490 ``tensor_raw``), with the
same error for an unknown name (crates/quant/src/error.rs:27-28).
"""
from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path

import numpy as np
import torch


class WeightFileError(ValueError):
    """A safetensors file that cannot be read: truncated, bad header, bad offsets."""


# safetensors dtype tag -> (torch dtype, bytes per element, numpy carrier dtype)
_DTYPES = {
    "F64": (torch.float64, 8, np.float64),
    "F32": (torch.float32, 4, np.float32),
    "F16": (torch.float16, 2, np.float16),
    "BF16": (torch.bfloat16, 2, np.uint16),
    "I64": (torch.int64, 8, np.int64),
    "I32": (torch.int32, 4, np.int32),
    "I16": (torch.int16, 2, np.int16),
    "I8": (torch.int8, 1, np.int8),
    "U8": (torch.uint8, 1, np.uint8),
    "BOOL": (torch.bool, 1, np.bool_),
}
_TAG_OF = {v[0]: k for k, v in _DTYPES.items()}


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: str            # safetensors tag, e.g. "BF16"
    shape: tuple
    begin: int
    end: int
    file: str

    @property
    def nbytes(self) -> int:
        return self.end - self.begin

    @property
    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n


class SafetensorsFile:
    """One memory-mapped safetensors file."""

    def __init__(self, path):
        self.path = Path(path)
        if not self.path.is_file():
            raise WeightFileError(f"{self.path}: no such file")
        size = self.path.stat().st_size
        if size < 8:
            raise WeightFileError(f"{self.path}: truncated (no header length)")
        self._fh = open(self.path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if 8 + hlen > size:
            raise WeightFileError(f"{self.path}: truncated (header of {hlen} bytes, file of {size})")
        try:
            header = json.loads(self._fh.read(hlen))
        except (json.JSONDecodeError, UnicodeDecodeError) as e:
            raise WeightFileError(f"{self.path}: header is not valid JSON ({e})") from e
        self._data_start = 8 + hlen
        data_len = size - self._data_start
        self.metadata = header.pop("__metadata__", None) or {}
        self.tensors: dict[str, TensorInfo] = {}
        spans = []
        for name, info in header.items():
            tag = info.get("dtype")
            if tag not in _DTYPES:
                raise WeightFileError(f"{self.path}: tensor '{name}' has unknown dtype {tag!r}")
            shape = tuple(int(s) for s in info["shape"])
            lo, hi = (int(x) for x in info["data_offsets"])
            ti = TensorInfo(name, tag, shape, lo, hi, str(self.path))
            if lo < 0 or hi < lo or hi > data_len:
                raise WeightFileError(
                    f"{self.path}: truncated: tensor '{name}' spans bytes {lo}..{hi} of {data_len}")
            if ti.numel * _DTYPES[tag][1] != hi - lo:
                raise WeightFileError(
                    f"{self.path}: tensor '{name}' of shape {list(shape)} and dtype {tag} needs "
                    f"{ti.numel * _DTYPES[tag][1]} bytes, header gives {hi - lo}")
            self.tensors[name] = ti
            if hi > lo:
                spans.append((lo, hi, name))
        spans.sort()
        for (lo0, hi0, n0), (lo1, hi1, n1) in zip(spans, spans[1:]):
            if lo1 < hi0:
                raise WeightFileError(f"{self.path}: tensors '{n0}' and '{n1}' overlap")
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self):
        return list(self.tensors)

    def info(self, name: str) -> TensorInfo:
        try:
            return self.tensors[name]
        except KeyError:
            raise KeyError(f"{self.path}: no tensor named '{name}'") from None

    def read(self, name: str) -> torch.Tensor:
        """A host tensor that owns its memory (a copy out of the map)."""
        ti = self.info(name)
        tdtype, _, carrier = _DTYPES[ti.dtype]
        lo = self._data_start + ti.begin
        arr = np.frombuffer(self._mm, dtype=carrier, count=ti.numel, offset=lo).copy()
        t = torch.from_numpy(arr)
        if ti.dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(ti.shape)

    def close(self):
        if self._mm is not None:
            self._mm.close()
            self._mm = None
        self._fh.close()


def write_safetensors(path, tensors, metadata: dict | None = None) -> None:
    """Write ``{name: host tensor}`` (a dict, or an iterable of pairs produced one at a
    time whose shapes are known up front through ``(name, shape, dtype, producer)``)."""
    items = list(tensors.items()) if isinstance(tensors, dict) else list(tensors)
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    plan = []
    for item in items:
        if len(item) == 2:
            name, t = item
            shape, dtype, producer = tuple(t.shape), t.dtype, (lambda t=t: t)
        else:
            name, shape, dtype, producer = item
        if dtype not in _TAG_OF:
            raise WeightFileError(f"cannot store tensor '{name}' of dtype {dtype}")
        tag = _TAG_OF[dtype]
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * _DTYPES[tag][1]
        header[name] = {"dtype": tag, "shape": [int(s) for s in shape],
                        "data_offsets": [offset, offset + nbytes]}
        plan.append((name, tuple(shape), dtype, producer, nbytes))
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype, producer, nbytes in plan:
            t = producer().detach().cpu().contiguous()
            if tuple(t.shape) != shape or t.dtype != dtype:
                raise WeightFileError(f"tensor '{name}' changed shape or dtype while being written")
            raw = t.view(torch.uint16) if dtype == torch.bfloat16 else t
            if dtype == torch.bool:
                raw = t.view(torch.uint8)
            data = raw.numpy().tobytes()
            assert len(data) == nbytes
            f.write(data)
