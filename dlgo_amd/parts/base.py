"""What every part of a model has in common.

A part owns tensors (declared by name and shape, relative to the prefix under
which the model mounts it), is given them once at load time, and runs on the
rows of a step.  It knows its own sizes and constants, never the model it sits
in.  computerex/dlgo keeps the same independence through per-layer enum choices
(models/llm/model.go:12-55) switched on in the forward pass
(models/llm/forward.go:142-182); here each choice is an object with one
interface per kind.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part expects: its shape, how it is stored, and how random
    weights are drawn for it.

    kind "matrix": operand of a matrix product, kept in the run dtype.
    kind "vector": per-channel weights (norms), kept in float32 (exact from bfloat16).
    kind "table":  integers, kept as int32.
    init "normal": N(0, std) with std the configuration's initializer range;
    init "ones":   1, or 1 + N(0, jitter) when the caller asks for jitter.
    """
    shape: Tuple[int, ...]
    kind: str = "matrix"
    init: str = "normal"


class Part:
    """Base of everything that may own tensors."""

    #: kernel modules (names under csrc/) this part launches; built before first use
    kernel_modules: Tuple[str, ...] = ()

    #: True if what the part launches for a step depends only on the step's device arrays and on its shape (the number of
    #: sequences, the rows each brings and the wanted places), so that the launches can be recorded once and replayed
    #: with new arrays: steps of single tokens per batch size, steps of fresh prompts per shape.  A part that reads the
    #: step's host-side numbers (ctx.host: lengths, slots) to decide what to launch or where to write, or launches
    #: through anything that cannot be recorded, sets this to False; a model with such a part runs every step, prompts
    #: included, as it is.
    graph_safe: bool = True

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor], device: torch.device, dtype: torch.dtype) -> None:
        """Take the tensors named in tensor_specs() (CPU, as stored) and keep them on
        `device` the way the kernels want them."""

    def check(self, dtype: torch.dtype) -> None:
        """Raise ValueError if the kernels of this part cannot take its sizes at `dtype` (called before anything runs)."""

    def takes_unscaled(self, ctx) -> bool:
        """True if, for this step, the part's forward also takes, in place of normed rows, the description of a norm
        whose factor is still to be applied (kernels.ops.UnscaledNorm: the rows times the norm's weights, and each
        row's sum of squares in shares).  The part that runs before may then leave the norm that way."""
        return False

    def kernel_variants(self, dtype: torch.dtype) -> Tuple[Tuple[str, Tuple[Tuple[str, int], ...]], ...]:
        """(module, defines) pairs to compile for this part at `dtype`."""
        from ..kernels.build import variant
        return tuple(variant(m, dtype) for m in self.kernel_modules)


def stored(t: torch.Tensor, spec: TensorSpec, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    """The storage rule: matrices in the run dtype, vectors in float32, tables in int32."""
    if spec.kind == "matrix":
        return t.to(device=device, dtype=dtype).contiguous()
    if spec.kind == "vector":
        return t.to(device=device, dtype=torch.float32).contiguous()
    if spec.kind == "table":
        return t.to(device=device, dtype=torch.int32).contiguous()
    raise ValueError(f"unknown tensor kind {spec.kind!r}")


@dataclass
class CacheNeed:
    """What a mixer asks of the cache for one run of a layer.

    kind "kv":    keys and values of every token (window None) or of the last
                  `window` tokens; kv_heads x head_dim each.
    kind "state": a fixed-size tensor per sequence (`state_shape`, `state_dtype`),
                  zero when a sequence starts.
    kind "none":  nothing.
    A mixer may ask for both keys/values and state by returning two needs.
    """
    kind: str = "none"
    kv_heads: int = 0
    head_dim: int = 0
    window: Optional[int] = None
    state_shape: Tuple[int, ...] = ()
    state_dtype: torch.dtype = torch.float32


def check_inner(what: str, sizes, dtype: torch.dtype) -> None:
    """The matrix products read 16 bytes at a time along their inner dimension."""
    per = 4 if dtype == torch.float32 else 8
    for name, n in sizes:
        if n % per:
            raise ValueError(f"{what}: {name} = {n} must be a multiple of {per} at {str(dtype).replace('torch.', '')} "
                             f"(the products load 16 bytes at a time)")
