"""Norms.  RMSNorm as computerex/dlgo computes it (ops/norm.go:10-32): no mean, no
bias, the weight multiplies as it is; the sum of squares and the scale are float32."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Part, TensorSpec, stored


class RMSNorm(Part):
    kernel_modules = ("rmsnorm",)

    def __init__(self, width: int, eps: float):
        self.width = width
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.width,), kind="vector", init="ones")}

    def load(self, tensors, device, dtype) -> None:
        self.weight = stored(tensors["weight"], self.tensor_specs()["weight"], device, dtype)

    def __call__(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """x: float32 rows of the residual stream; out: rows in the run dtype (gathered by `rows` if given)."""
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)


NORMS = {"rmsnorm": RMSNorm}
