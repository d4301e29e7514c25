"""Weights by tensor name.

The model says which tensors it expects and with what shapes; the file says which
it has.  Every disagreement is collected into one error: missing tensors,
unexpected tensors, wrong shapes, unsupported types.  computerex/dlgo routes each
tensor of the file by name (models/llm/loader.go:47-71,168-262), ignores names it
does not know and does not notice missing ones (a test looks for nil fields,
models/llm/e2e_test.go:497-525); here both are errors.

Storage: operands of matrix products in the run dtype, norm weights in float32
(a bfloat16 value widens exactly; a tensor the file holds in 32-bit is never
narrowed unless it is a matrix-product operand of a bfloat16 run), integer
tables as int32.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile, TensorInfo

_FLOAT_TYPES = ("BF16", "F16", "F32")
_INT_TYPES = ("I64", "I32", "I16", "I8", "U8")


class WeightsError(ValueError):
    """One error for everything wrong between a model and a weights folder."""

    def __init__(self, where: str, missing=(), unexpected=(), wrong_shape=(), wrong_type=(), other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_type, self.other = list(wrong_shape), list(wrong_type), list(other)
        lines = [f"{where}: weights do not match the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, found in self.wrong_shape:
            lines.append(f"  wrong shape: {name} expected {list(want)}, found {list(found)}")
        for name, found in self.wrong_type:
            lines.append(f"  unsupported type: {name} is {found}")
        lines.extend(f"  {o}" for o in self.other)
        super().__init__("\n".join(lines))


def open_folder(folder: str) -> Dict[str, SafetensorsFile]:
    """tensor name -> the open file that holds it (model.safetensors, or the shards of an index)."""
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    files: List[str]
    if os.path.exists(single):
        files = [single]
    elif os.path.exists(index):
        with open(index) as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
        outside = [v for v in shards if not isinstance(v, str) or os.path.isabs(v) or os.path.basename(v) != v or v in ("", ".", "..")]
        if outside:
            raise WeightsError(folder, other=[f"the index names a shard outside the folder: {v!r}" for v in outside])
        files = [os.path.join(folder, v) for v in shards]
    else:
        raise WeightsError(folder, other=[f"neither model.safetensors nor model.safetensors.index.json found"])
    where: Dict[str, SafetensorsFile] = {}
    dup = []
    for path in files:
        try:
            sf = SafetensorsFile(path)
        except SafetensorsError as e:
            raise WeightsError(folder, other=[str(e)]) from None
        for name in sf.infos:
            if name in where:
                dup.append(f"duplicate tensor {name} in {os.path.basename(where[name].path)} and {os.path.basename(path)}")
            where[name] = sf
    if dup:
        raise WeightsError(folder, other=dup)
    return where


def check(model, infos: Dict[str, TensorInfo], where: str) -> None:
    expected = model.expected_tensors()
    missing = [n for n in expected if n not in infos]
    unexpected = [n for n in infos if n not in expected and n not in model.ignorable_tensors]
    wrong_shape, wrong_type = [], []
    for name, spec in expected.items():
        if name not in infos:
            continue
        info = infos[name]
        if tuple(info.shape) != tuple(spec.shape):
            wrong_shape.append((name, spec.shape, info.shape))
        ok = _INT_TYPES if spec.kind == "table" else _FLOAT_TYPES
        if info.dtype not in ok:
            wrong_type.append((name, info.dtype))
    if missing or unexpected or wrong_shape or wrong_type:
        raise WeightsError(where, missing, unexpected, wrong_shape, wrong_type)


def load_weights(model, folder: str, device, dtype: torch.dtype) -> None:
    """Read every tensor the model expects from `folder` and hand each part its own."""
    files = open_folder(folder)
    check(model, {n: f.infos[n] for n, f in files.items()}, folder)
    device = torch.device(device)
    for prefix, part in model.named_parts():
        specs = part.tensor_specs()
        try:
            tensors = {name: files[f"{prefix}.{name}"].tensor(f"{prefix}.{name}") for name in specs}
        except SafetensorsError as e:
            raise WeightsError(folder, other=[str(e)]) from None
        part.load(tensors, device, dtype)
    for f in set(files.values()):
        f.close()


def load_state(model, tensors: Dict[str, torch.Tensor], device, dtype: torch.dtype, where: str = "tensors") -> None:
    """The same, from tensors already in memory (random weights that were never written)."""
    infos = {}
    names = {torch.bfloat16: "BF16", torch.float16: "F16", torch.float32: "F32", torch.int32: "I32", torch.int64: "I64"}
    for n, t in tensors.items():
        infos[n] = TensorInfo(n, names.get(t.dtype, str(t.dtype)), tuple(t.shape), 0, 0, where)
    check(model, infos, where)
    device = torch.device(device)
    for prefix, part in model.named_parts():
        part.load({name: tensors[f"{prefix}.{name}"] for name in part.tensor_specs()}, device, dtype)
