"""Random weights from a configuration and a seed, in memory or as a model folder.

computerex/dlgo has nothing of the kind for language models; its fixture
generator draws random speech models from a seeded stream, tensor after tensor
(testdata/generate.go:45-148), so a value there depends on every draw before it.
Here a value depends on three numbers only, the seed, the tensor's name and the
element's index, so anyone can compute any element without the others:

    key      = splitmix64(seed XOR fnv1a64(name))
    draw(c)  = splitmix64(key + c * 0x9E3779B97F4A7C15)              (64 bits, c = 1, 2, ...)
    u(c)     = ((draw(c) >> 11) + 1) / 2^53                          (float64 in (0, 1])
    normal i = sqrt(-2 ln u(2i + 1)) * cos(2 pi u(2i + 2))           (Box-Muller in float64)

A matrix or table element is float32(normal * std), a norm weight 1 or
float32(1 + normal * norm_jitter) when asked (so that a norm applied in the wrong
place, or as 1 + w, shows), each then rounded to the stored type (bfloat16: to
nearest, ties to even).  The arithmetic runs on the host in NumPy float64,
whatever device the tensors then go to, so a model drawn straight onto the GPU
and a model folder written for the same seed hold the same bits.  An integer
table holds, in each row, the permutation that sorts that row's draws.
"""
from __future__ import annotations

import json
import math
import os
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Optional

import numpy as np
import torch

from ..config import ModelConfig, build_model
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}
_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_CHUNK = 1 << 20          # elements drawn at a time by one worker


def _mix(z: int) -> int:
    """splitmix64's output function on a Python integer."""
    z &= _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def tensor_key(seed: int, name: str) -> int:
    h = 0xCBF29CE484222325
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 0x100000001B3) & _MASK
    return _mix((int(seed) & _MASK) ^ h)


def _mix_in_place(z: np.ndarray, t: np.ndarray) -> None:
    """splitmix64's output function on every element of z (uint64); t is scratch of the same shape."""
    np.right_shift(z, np.uint64(30), out=t)
    np.bitwise_xor(z, t, out=z)
    np.multiply(z, np.uint64(0xBF58476D1CE4E5B9), out=z)
    np.right_shift(z, np.uint64(27), out=t)
    np.bitwise_xor(z, t, out=z)
    np.multiply(z, np.uint64(0x94D049BB133111EB), out=z)
    np.right_shift(z, np.uint64(31), out=t)
    np.bitwise_xor(z, t, out=z)


def _draws(key: int, first: int, count: int, step: int = 1) -> np.ndarray:
    """draw(first), draw(first + step), ... (count of them) as uint64."""
    z = np.arange(count, dtype=np.uint64)
    np.multiply(z, np.uint64((step * _GOLDEN) & _MASK), out=z)
    np.add(z, np.uint64((key + first * _GOLDEN) & _MASK), out=z)
    _mix_in_place(z, np.empty_like(z))
    return z


def _unit(d: np.ndarray) -> np.ndarray:
    """uint64 draws -> float64 in (0, 1]."""
    np.right_shift(d, np.uint64(11), out=d)
    u = d.astype(np.float64)
    np.add(u, 1.0, out=u)
    np.multiply(u, 1.0 / 9007199254740992.0, out=u)
    return u


def _normals(key: int, first: int, count: int) -> np.ndarray:
    """Standard normals of elements first .. first + count - 1, float64: element i from draws 2i + 1 and 2i + 2."""
    r = _unit(_draws(key, 2 * first + 1, count, 2))
    np.log(r, out=r)
    np.multiply(r, -2.0, out=r)
    np.sqrt(r, out=r)
    a = _unit(_draws(key, 2 * first + 2, count, 2))
    np.multiply(a, 2.0 * math.pi, out=a)
    np.cos(a, out=a)
    np.multiply(r, a, out=r)
    return r


_pool: Optional[ThreadPoolExecutor] = None


def _workers() -> ThreadPoolExecutor:
    global _pool
    if _pool is None:
        _pool = ThreadPoolExecutor(max_workers=max(1, min(16, os.cpu_count() or 1)))
    return _pool


def normal_tensor(seed: int, name: str, shape, scale: float, offset: float = 0.0) -> torch.Tensor:
    """float32 tensor of `shape` with element i (row-major) = float32(offset + scale * normal i of (seed, name))."""
    n = math.prod(shape)
    out = np.empty(n, dtype=np.float32)
    key = tensor_key(seed, name)

    def fill(start: int) -> None:
        count = min(_CHUNK, n - start)
        v = _normals(key, start, count)
        np.multiply(v, scale, out=v)
        if offset:
            np.add(v, offset, out=v)
        out[start:start + count] = v          # float64 -> float32, to nearest

    starts = range(0, n, _CHUNK)
    if n > _CHUNK:
        list(_workers().map(fill, starts))
    else:
        for s0 in starts:
            fill(s0)
    return torch.from_numpy(out).reshape(tuple(shape))


def _table(seed: int, name: str, spec) -> torch.Tensor:
    """An integer table: in every row the permutation of its last axis that sorts the row's draws (ids that stay inside
    the table's own range, whatever they index)."""
    rows, width = math.prod(spec.shape[:-1]), spec.shape[-1]
    d = _draws(tensor_key(seed, name), 1, rows * width).reshape(rows, width)
    return torch.from_numpy(np.argsort(d, axis=-1, kind="stable").astype(np.int32)).reshape(tuple(spec.shape))


def random_tensors(config: ModelConfig, seed: int, dtype: Optional[torch.dtype] = None, std: Optional[float] = None,
                   norm_jitter: float = 0.0, device="cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor for every tensor the architecture expects.  Values are drawn in float64, stored as float32 and
    rounded to `dtype` (default: the type the configuration says its checkpoints have), norm weights included, as a
    checkpoint of that type holds them."""
    model = build_model(config)
    if dtype is None:
        dtype = _DTYPES[config.storage_dtype()]
    if std is None:
        std = config.init_std()
        if std is None:
            raise ValueError("random weights: the configuration names no standard deviation (initializer_range); pass std")
    out: Dict[str, torch.Tensor] = {}
    for name, spec in model.expected_tensors().items():
        if spec.kind == "table":
            out[name] = _table(seed, name, spec).to(device)
            continue
        if spec.init == "ones":
            t = normal_tensor(seed, name, spec.shape, norm_jitter, 1.0) if norm_jitter else torch.ones(spec.shape, dtype=torch.float32)
        elif spec.init == "normal":
            t = normal_tensor(seed, name, spec.shape, std)
        else:
            raise ValueError(f"random weights: unknown init {spec.init!r} of {name}")
        out[name] = t.to(dtype).to(device)
    return out


def write_random_model(config: ModelConfig, seed: int, folder: str, dtype: Optional[torch.dtype] = None,
                       std: Optional[float] = None, norm_jitter: float = 0.0) -> str:
    """Write config.json and model.safetensors for `config` into `folder`."""
    os.makedirs(folder, exist_ok=True)
    tensors = random_tensors(config, seed, dtype, std, norm_jitter)
    if dtype is not None:
        config = config.stored_as({v: k for k, v in _DTYPES.items()}[dtype])
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return folder
