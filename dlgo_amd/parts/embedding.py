"""Token embedding and output head.  The embedding copies a table row per token,
unscaled (computerex/dlgo, models/llm/forward.go:132-135); the head multiplies the
normed rows by the output matrix, which is the embedding table when the model
ties them (models/llm/loader.go:74-76; forward.go:193-201), into float32 logits."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Part, TensorSpec, check_inner, stored
from .norm import RMSNorm


class Embedding(Part):
    kernel_modules = ("embed",)

    def __init__(self, vocab: int, width: int):
        self.vocab, self.width = vocab, width
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab, self.width))}

    def load(self, tensors, device, dtype) -> None:
        self.weight = stored(tensors["weight"], self.tensor_specs()["weight"], device, dtype)

    def __call__(self, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        return ops.embed(self.weight, ids, out)


class OutputHead(Part):
    kernel_modules = ("gemm", "gemm_rows")

    def __init__(self, vocab: int, width: int, tied_to: Optional[Embedding] = None):
        self.vocab, self.width = vocab, width
        self.tied_to = tied_to
        self._weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {} if self.tied_to is not None else {"weight": TensorSpec((self.vocab, self.width))}

    def load(self, tensors, device, dtype) -> None:
        if self.tied_to is None:
            self._weight = stored(tensors["weight"], self.tensor_specs()["weight"], device, dtype)

    def check(self, dtype) -> None:
        check_inner("output head", (("width", self.width),), dtype)

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def fuses_norm(self, norm, ctx) -> bool:
        return isinstance(norm, RMSNorm) and ops.fused_norm_pays(self.weight, ctx.n_tokens)

    def takes_unscaled(self, ctx) -> bool:
        return ops.streams_few_rows(self.weight, ctx.n_tokens, ops.ROLE_APPLIES_NORM)

    def __call__(self, xn, out: torch.Tensor, norm=None) -> torch.Tensor:
        """xn: normed rows (run dtype), or what stands for them (see Part.takes_unscaled), or with `norm` the float32
        residual rows; out: float32 [rows, vocab]."""
        if isinstance(xn, ops.UnscaledNorm):
            return ops.gemm_scaled(self.weight, xn, out, ops.EPI_STORE_F32)
        if norm is not None:
            return ops.gemm_rmsnorm(self.weight, xn, norm.weight, norm.eps, out, ops.EPI_STORE_F32)
        return ops.gemm(self.weight, xn, out, ops.EPI_STORE_F32)
