"""Parts of a model and the registries that map a kind's name to its class.

A new mixer, feed-forward, norm, position encoding or block arrangement is added
by writing a class with the kind's interface and registering it; architectures
choose parts by these names, layer by layer.
"""
from .attention import Attention, Mixer
from .base import CacheNeed, Part, TensorSpec, stored
from .block import BLOCKS, Block, PreNormBlock
from .embedding import Embedding, OutputHead
from .feed_forward import FeedForward, GatedFeedForward
from .model import DecoderModel, LayerRun
from .norm import NORMS, RMSNorm
from .position import POSITIONS, NoPosition, PositionEncoding, Rotary, Rotation, rotary_frequencies

MIXERS = {"attention": Attention}
FEED_FORWARDS = {"gated": GatedFeedForward}

_KINDS = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "position": POSITIONS, "block": BLOCKS}


def register_part(kind: str, name: str, cls) -> None:
    """kind: one of mixer, feed_forward, norm, position, block."""
    if kind not in _KINDS:
        raise ValueError(f"unknown kind of part {kind!r}; kinds: {', '.join(_KINDS)}")
    _KINDS[kind][name] = cls


def make_part(kind: str, name: str, *args, **kwargs):
    if kind not in _KINDS:
        raise ValueError(f"unknown kind of part {kind!r}; kinds: {', '.join(_KINDS)}")
    if name not in _KINDS[kind]:
        raise ValueError(f"unknown {kind} {name!r}; known: {', '.join(sorted(_KINDS[kind]))}")
    return _KINDS[kind][name](*args, **kwargs)


__all__ = ["Attention", "Mixer", "CacheNeed", "Part", "TensorSpec", "stored", "Block", "PreNormBlock", "Embedding",
           "OutputHead", "FeedForward", "GatedFeedForward", "DecoderModel", "LayerRun", "RMSNorm", "NoPosition",
           "PositionEncoding", "Rotary", "Rotation", "rotary_frequencies", "MIXERS", "FEED_FORWARDS", "NORMS",
           "POSITIONS", "BLOCKS", "register_part", "make_part"]
