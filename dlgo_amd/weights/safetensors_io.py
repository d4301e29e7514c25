"""Reading and writing safetensors files: an 8-byte little-endian header length,
a JSON header {name: {dtype, shape, data_offsets}}, then the raw bytes.

This stands where computerex/dlgo's GGUF parser stands (format/gguf/gguf.go:132-271):
it yields tensor names, shapes, types and a data offset, and reads nothing else.
Tensors are memory-mapped, so a large file is never held twice.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Mapping, Tuple

import torch

_DTYPES = {
    "BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorInfo:
    name: str
    dtype: str                 # the file's own word, e.g. "BF16"
    shape: Tuple[int, ...]
    begin: int
    end: int
    file: str


class SafetensorsFile:
    """One open file: `infos` by name, `tensor(name)` as a CPU tensor over the mapping."""

    def names(self):
        return list(self.infos)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            self._f = open(path, "rb")
        except OSError as e:
            raise SafetensorsError(f"{path}: {e.strerror or e}") from None
        head = self._f.read(8)
        if len(head) < 8:
            raise SafetensorsError(f"{path}: truncated (no header length)")
        (hlen,) = struct.unpack("<Q", head)
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: truncated (header of {hlen} bytes does not fit in {size})")
        try:
            header = json.loads(self._f.read(hlen))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self.data_start = 8 + hlen
        self.infos: Dict[str, TensorInfo] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                b, e = (int(v) for v in info["data_offsets"])
                shape = tuple(int(s) for s in info["shape"])
                dtype_name = info["dtype"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: header entry of tensor {name} is malformed") from None
            if b < 0 or e < b or any(d < 0 for d in shape):
                raise SafetensorsError(f"{path}: tensor {name} has offsets [{b}, {e}) and shape {list(shape)}")
            if self.data_start + e > size:
                raise SafetensorsError(f"{path}: truncated (tensor {name} ends at byte {self.data_start + e} of {size})")
            if dtype_name in _DTYPES:
                n = 1
                for d in shape:
                    n *= d
                want = n * torch.empty(0, dtype=_DTYPES[dtype_name]).element_size()
                if e - b != want:
                    raise SafetensorsError(f"{path}: tensor {name} of shape {list(shape)} and type {dtype_name} needs {want} bytes, "
                                           f"its offsets [{b}, {e}) give {e - b}")
            self.infos[name] = TensorInfo(name, info["dtype"], shape, b, e, path)
        self._map = None

    def tensor(self, name: str) -> torch.Tensor:
        info = self.infos[name]
        if info.dtype not in _DTYPES:
            raise SafetensorsError(f"{self.path}: tensor {name} has unsupported dtype {info.dtype}")
        dt = _DTYPES[info.dtype]
        n = 1
        for s in info.shape:
            n *= s
        if n == 0:
            return torch.empty(info.shape, dtype=dt)
        if self._map is None:
            self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")   # torch warns that the mapping is read-only; nothing writes to it
            t = torch.frombuffer(self._map, dtype=dt, count=n, offset=self.data_start + info.begin)
        return t.reshape(info.shape)

    def close(self) -> None:
        # tensors handed out keep the mapping alive; only the descriptor is closed here
        try:
            self._f.close()
        except OSError:
            pass


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor] | Iterable[Tuple[str, torch.Tensor]],
                      metadata: Mapping[str, str] | None = None) -> None:
    """Write tensors (CPU, contiguous) in the order given."""
    items = list(tensors.items()) if isinstance(tensors, Mapping) else list(tensors)
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    for name, t in items:
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot write {name}: dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in items:
            t = t.detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
