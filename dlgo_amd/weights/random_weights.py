"""Random weights from a configuration and a seed, in memory or as a model folder.

computerex/dlgo has nothing of the kind for language models (its fixture
generator writes random speech models, testdata/generate.go:45-148).  Each tensor
is drawn from a generator keyed by (seed, tensor name), so a tensor's values do
not depend on which other tensors exist: matrices and tables N(0, std) with std
the configuration's initializer_range unless given, norm weights 1, or
1 + N(0, norm_jitter) when asked (so that a norm applied in the wrong place, or
as 1 + w, shows).
"""
from __future__ import annotations

import json
import math
import os
import zlib
from typing import Dict, Optional

import torch

from ..config import ModelConfig, build_model
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _generator(seed: int, name: str) -> torch.Generator:
    """A tensor's own stream, keyed by the seed and the tensor's name.  It always runs on the host, so that a model drawn
    straight onto a device and a model folder written for the same seed hold the same values."""
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    return g


def _table(spec, g: torch.Generator) -> torch.Tensor:
    """An integer table: a random permutation of its last axis in every row (ids that stay inside the table's own range,
    whatever they index)."""
    rows = math.prod(spec.shape[:-1])
    perms = torch.stack([torch.randperm(spec.shape[-1], generator=g) for _ in range(rows)])
    return perms.reshape(spec.shape).to(torch.int32)


def random_tensors(config: ModelConfig, seed: int, dtype: Optional[torch.dtype] = None, std: Optional[float] = None,
                   norm_jitter: float = 0.0, device="cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor for every tensor the architecture expects.  Values are drawn in float32 and
    rounded to `dtype` (default: the configuration's torch_dtype), norm weights included, as a
    checkpoint of that type holds them."""
    model = build_model(config)
    if dtype is None:
        dtype = _DTYPES[getattr(config, "torch_dtype", "bfloat16")]
    if std is None:
        std = getattr(config, "initializer_range", None)
        if std is None:
            raise ValueError("random weights: the configuration has no initializer_range; pass std")
    out: Dict[str, torch.Tensor] = {}
    for name, spec in model.expected_tensors().items():
        g = _generator(seed, name)
        if spec.kind == "table":
            out[name] = _table(spec, g).to(device)
            continue
        if spec.init == "ones":
            t = torch.ones(spec.shape, dtype=torch.float32)
            if norm_jitter:
                t += norm_jitter * torch.randn(spec.shape, generator=g, dtype=torch.float32)
        elif spec.init == "normal":
            t = torch.randn(spec.shape, generator=g, dtype=torch.float32) * std
        else:
            raise ValueError(f"random weights: unknown init {spec.init!r} of {name}")
        out[name] = t.to(dtype).to(device)
    return out


def write_random_model(config: ModelConfig, seed: int, folder: str, dtype: Optional[torch.dtype] = None,
                       std: Optional[float] = None, norm_jitter: float = 0.0) -> str:
    """Write config.json and model.safetensors for `config` into `folder`."""
    os.makedirs(folder, exist_ok=True)
    tensors = random_tensors(config, seed, dtype, std, norm_jitter)
    raw = config.to_dict()
    if dtype is not None:
        raw["torch_dtype"] = {v: k for k, v in _DTYPES.items()}[dtype]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return folder
