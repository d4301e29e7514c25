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
    forward(x, ctx, unit, owns_cache) updates the float32 residual rows x in place.

    A block that sets `takes_normed` has an `entry_norm` (the norm it applies to x first) and a forward that also takes
    normed= (rows that already hold entry_norm(x), left by the block before, or what that block returned in their
    place) and then=(the next block's entry norm, rows, the part that will read them), and returns True if it left that
    norm of its result in `rows`, or what its last part left instead (see Mixer)."""
    takes_normed = False

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

    takes_normed = True

    @property
    def entry_norm(self) -> Part:
        return self.mixer_norm

    def forward(self, x, ctx, unit, owns_cache=True, normed=None, then=None):
        xn = ctx.buffer("block.normed", tuple(x.shape), ctx.dtype)
        # the mixer may leave the feed-forward's norm of its result, the feed-forward the next block's entry norm
        after = (self.ffn_norm, xn, self.ffn) if self._mixer.leaves_norm else None
        if normed is not None:
            left = self._mixer.forward(normed, ctx, unit, x, owns_cache, **({"then": after} if after else {}))
        elif self._mixer.fuses_norm(self.mixer_norm, ctx):
            left = self._mixer.forward(x, ctx, unit, x, owns_cache, norm=self.mixer_norm, **({"then": after} if after else {}))
        else:
            self.mixer_norm(x, xn)
            # the mixer reads xn until its last product, whose sum is what writes the norm: a buffer of its own
            mid = ctx.buffer("block.normed_mid", tuple(x.shape), ctx.dtype) if after else None
            if after:
                after = (self.ffn_norm, mid, self.ffn)
            left = self._mixer.forward(xn, ctx, unit, x, owns_cache, **({"then": after} if after else {}))
            if left:
                xn = mid
        onward = {"then": then} if then is not None and self.ffn.leaves_norm else {}
        if left:       # True: the rows hold the norm; anything else stands for them
            return self.ffn.forward(xn if left is True else left, ctx, x, **onward) or False
        if self.ffn.fuses_norm(self.ffn_norm, ctx):
            return self.ffn.forward(x, ctx, x, norm=self.ffn_norm, **onward) or False
        self.ffn_norm(x, xn)
        return self.ffn.forward(xn, ctx, x, **onward) or False


BLOCKS = {"pre_norm": PreNormBlock}
