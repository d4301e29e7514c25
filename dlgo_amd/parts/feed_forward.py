"""Feed-forward parts.  The gated one is SwiGLU as computerex/dlgo computes it
(models/llm/forward.go:295-298; ops/activation.go:8-19,36-38): hid = silu(gate x) * (up x),
out = down hid, no biases.  Gate and up rows are interleaved at load, so one matrix
product yields both and its epilogue writes `hid` once; the down projection adds
into the float32 residual stream."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Part, TensorSpec, check_inner, stored
from .norm import RMSNorm


class FeedForward(Part):
    """Interface: forward(xn, ctx, residual) adds the result for the step's rows into `residual`.  One that sets
    `leaves_norm` also takes then=(norm part, rows[, the part that will read them]) and returns True if it left that
    norm of the new residual rows in `rows`, or what it left instead (see Mixer)."""
    leaves_norm = False

    def fuses_norm(self, norm, ctx) -> bool:
        """True if, for this step, it would rather be given the float32 residual rows and the norm part."""
        return False

    def forward(self, xn: torch.Tensor, ctx, residual: torch.Tensor, norm=None) -> None:
        raise NotImplementedError


class GatedFeedForward(FeedForward):
    kernel_modules = ("gemm", "gemm_rows")
    leaves_norm = True

    def __init__(self, width: int, inner: int, activation: str = "silu"):
        if activation != "silu":
            raise ValueError(f"gated feed-forward: activation {activation!r} has no kernel (silu has)")
        self.width, self.inner = width, inner
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            "gate_proj.weight": TensorSpec((self.inner, self.width)),
            "up_proj.weight": TensorSpec((self.inner, self.width)),
            "down_proj.weight": TensorSpec((self.width, self.inner)),
        }

    def check(self, dtype) -> None:
        check_inner("feed-forward", (("width", self.width), ("inner width", self.inner)), dtype)

    def load(self, tensors, device, dtype) -> None:
        spec = self.tensor_specs()
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        inter = torch.stack([gate, up], dim=1).reshape(2 * self.inner, self.width)   # rows g0,u0,g1,u1,...
        self.w_gate_up = stored(inter, spec["gate_proj.weight"], device, dtype)
        self.w_down = stored(tensors["down_proj.weight"], spec["down_proj.weight"], device, dtype)

    def fuses_norm(self, norm, ctx) -> bool:
        return isinstance(norm, RMSNorm) and ops.fused_norm_pays(self.w_gate_up, ctx.n_tokens)

    def takes_unscaled(self, ctx) -> bool:
        return ops.can_take_unscaled(self.w_gate_up, ctx.n_tokens)

    def forward(self, xn, ctx, residual, norm=None, then=None):
        hid = ctx.buffer("feed_forward.hidden", (residual.shape[0], self.inner), ctx.dtype)
        if isinstance(xn, ops.UnscaledNorm):   # the norm's factor is applied to the product's sums
            ops.gemm_scaled(self.w_gate_up, xn, hid, ops.EPI_SWIGLU)
        elif norm is not None:    # xn are the float32 residual rows: the norm rides in the product
            ops.gemm_rmsnorm(self.w_gate_up, xn, norm.weight, norm.eps, hid, ops.EPI_SWIGLU)
        else:
            ops.gemm(self.w_gate_up, xn, hid, ops.EPI_SWIGLU)
        split = ctx.scratch("gemm.split", ops.GEMM_SPLIT_FLOATS, torch.float32)
        if then is not None and isinstance(then[0], RMSNorm):
            if ops.gemm_accum_then_norm(self.w_down, hid, residual, split, then[0].weight, then[0].eps, then[1]):
                return True
            # many rows: the tiled product leaves the norm unscaled, if what reads it can apply the factor (with few rows
            # the split product and its sum above are as fast as the streamed product that would leave it)
            t = residual.shape[0]
            if t > 16 and len(then) > 2 and then[2] is not None and then[2].takes_unscaled(ctx) \
                    and ops.can_leave_unscaled(self.w_down, t):
                shares = ctx.scratch("feed_forward.norm_shares", t * ((self.width + 7) // 8), torch.float32)
                return ops.gemm_accum_leave_norm(self.w_down, hid, residual, then[0].weight, then[0].eps, then[1], shares)
        ops.gemm(self.w_down, hid, residual, ops.EPI_ACCUM_F32, scratch=split)
        return False
