"""How the parts of one layer are arranged.  PreNormBlock is the wiring
computerex/dlgo calls ResStandard (models/llm/model.go:28-34; forward.go:144-169):
x += mixer(norm(x)); x += feed_forward(norm(x)), both sums in float32."""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from .attention import Mixer
from .base import Part
from .feed_forward import FeedForward


class Block(Part):
    """Interface: parts() names the sub-parts (the names become tensor-name prefixes);
    forward(x, ctx, unit, owns_cache) updates the float32 residual rows x in place."""

    def parts(self) -> List[Tuple[str, Part]]:
        raise NotImplementedError

    @property
    def mixer(self) -> Mixer:
        raise NotImplementedError

    def forward(self, x: torch.Tensor, ctx, unit: int, owns_cache: bool = True) -> None:
        raise NotImplementedError


class PreNormBlock(Block):
    def __init__(self, mixer_norm: Tuple[str, Part], mixer: Tuple[str, Mixer], ffn_norm: Tuple[str, Part],
                 ffn: Tuple[str, FeedForward]):
        self._parts = [mixer_norm, mixer, ffn_norm, ffn]
        self.mixer_norm, self._mixer, self.ffn_norm, self.ffn = mixer_norm[1], mixer[1], ffn_norm[1], ffn[1]

    def parts(self):
        return list(self._parts)

    @property
    def mixer(self) -> Mixer:
        return self._mixer

    def forward(self, x, ctx, unit, owns_cache=True) -> None:
        xn = ctx.buffer("block.normed", tuple(x.shape), ctx.dtype)
        if self._mixer.fuses_norm(self.mixer_norm, ctx):
            self._mixer.forward(x, ctx, unit, x, owns_cache, norm=self.mixer_norm)
        else:
            self.mixer_norm(x, xn)
            self._mixer.forward(xn, ctx, unit, x, owns_cache)
        if self.ffn.fuses_norm(self.ffn_norm, ctx):
            self.ffn.forward(x, ctx, x, norm=self.ffn_norm)
        else:
            self.ffn_norm(x, xn)
            self.ffn.forward(xn, ctx, x)


BLOCKS = {"pre_norm": PreNormBlock}
