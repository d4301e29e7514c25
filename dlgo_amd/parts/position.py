"""Position encodings.

Rotary: pair i of a head turns by the angle pos * theta_i, theta_i =
base^(-2i/width) (computerex/dlgo, ops/rope.go:13-33); cos and sin come from a
table computed in float64 and stored as float32, one row per position
(models/llm/workers.go:147-171).  The llama3 scaling of the frequencies has no
counterpart in the reference: wavelengths shorter than P0/high keep their
frequency, longer than P0/low have it divided by the factor, and those between
are blended linearly in (P0/wavelength - low)/(high - low).

A position encoding offers two hooks: `on_embedding` (something added to the
embedded rows; nothing for rotary) and `rotation` (tables for the fused
rotate-and-store kernel of an attention mixer; None if it rotates nothing).
"""
from __future__ import annotations

import math
import weakref
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .base import Part


@dataclass
class Rotation:
    cos: torch.Tensor        # [positions, width/2] float32
    sin: torch.Tensor
    width: int               # rotated width of a head (<= head size)
    interleaved: bool


class PositionEncoding(Part):
    def prepare(self, max_positions: int, device: torch.device) -> None:
        """Build whatever tables the encoding needs for positions below max_positions."""

    def on_embedding(self, x: torch.Tensor, ctx) -> None:
        """Add a position term to the embedded rows (float32, in place)."""

    def rotation(self) -> Optional[Rotation]:
        return None


class NoPosition(PositionEncoding):
    pass


def rotary_frequencies(width: int, theta: float, scaling=None) -> np.ndarray:
    """theta_i for i in [0, width/2), float64, with the llama3 recipe applied if given
    (an object with factor, low_freq_factor, high_freq_factor, original_max_position_embeddings)."""
    half = width // 2
    freq = np.array([1.0 / math.pow(float(theta), (2.0 * i) / width) for i in range(half)], dtype=np.float64)
    if scaling is None:
        return freq
    f, lo, hi = float(scaling.factor), float(scaling.low_freq_factor), float(scaling.high_freq_factor)
    p0 = float(scaling.original_max_position_embeddings)
    out = freq.copy()
    for i in range(half):
        wavelength = 2.0 * math.pi / freq[i]
        if wavelength < p0 / hi:
            continue
        if wavelength > p0 / lo:
            out[i] = freq[i] / f
        else:
            s = (p0 / wavelength - lo) / (hi - lo)
            out[i] = (1.0 - s) * freq[i] / f + s * freq[i]
    return out


class _Tables:
    """cos and sin of position * frequency for one recipe of frequencies, [positions, width/2] float32 each."""
    __slots__ = ("cos", "sin", "__weakref__")

    def __init__(self, cos: torch.Tensor, sin: torch.Tensor):
        self.cos, self.sin = cos, sin


# One pair of tables per distinct recipe (the frequencies themselves, which theta, width and scaling determine) and device,
# shared by every layer that names the recipe: a model of 16 equal layers holds one, and a decode step reads one.  The
# entries live as long as a part holds them.
_TABLES: "weakref.WeakValueDictionary[tuple, _Tables]" = weakref.WeakValueDictionary()


def rotary_tables(frequencies: np.ndarray, max_positions: int, device: torch.device) -> _Tables:
    key = (frequencies.tobytes(), str(torch.device(device)))
    held = _TABLES.get(key)
    if held is not None and held.cos.shape[0] >= max_positions:
        return held
    angles = np.arange(max_positions, dtype=np.float64)[:, None] * frequencies[None, :]
    cos = torch.from_numpy(np.cos(angles).astype(np.float32)).to(device)
    sin = torch.from_numpy(np.sin(angles).astype(np.float32)).to(device)
    held = _Tables(cos.contiguous(), sin.contiguous())
    _TABLES[key] = held          # longer tables take the shorter ones' place for whoever asks next
    return held


class Rotary(PositionEncoding):
    kernel_modules = ("rope_kv",)

    def __init__(self, head_dim: int, theta: float, scaling=None, width: Optional[int] = None, interleaved: bool = False):
        self.head_dim = head_dim
        self.width = head_dim if width is None else width
        if self.width % 2 or not 0 < self.width <= head_dim:
            raise ValueError(f"rotary: rotated width {self.width} must be even and at most the head size {head_dim}")
        self.theta = float(theta)
        self.scaling = scaling
        self.interleaved = interleaved
        self.frequencies = rotary_frequencies(self.width, self.theta, scaling)
        self._tables: Optional[_Tables] = None
        self._rotation: Optional[Rotation] = None

    def prepare(self, max_positions: int, device: torch.device) -> None:
        if self._rotation is not None and self._rotation.cos.shape[0] >= max_positions and self._rotation.cos.device == torch.device(device):
            return
        self._tables = rotary_tables(self.frequencies, max_positions, device)
        self._rotation = Rotation(self._tables.cos, self._tables.sin, self.width, self.interleaved)

    def rotation(self) -> Optional[Rotation]:
        if self._rotation is None:
            raise RuntimeError("rotary tables are built by prepare() before the first step")
        return self._rotation


POSITIONS = {"rotary": Rotary, "none": NoPosition}
