"""Uniform numbers for the draws: one stream per request, keyed by (seed, request
index, step), so a request's samples do not depend on its batch-mates.
computerex/dlgo uses one math/rand stream per call (models/llm/generate.go:92-95);
seed < 0 takes the clock there and here."""
from __future__ import annotations

import time

_MASK = (1 << 64) - 1


def _mix(x: int) -> int:
    """splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def resolve_seed(seed: int) -> int:
    return seed if seed >= 0 else time.time_ns() & 0x7FFFFFFFFFFFFFFF


def uniform(seed: int, request: int, step: int) -> float:
    """A float32-representable number in [0, 1)."""
    h = _mix(_mix(_mix(seed & _MASK) ^ (request & _MASK)) ^ (step & _MASK))
    return (h >> 40) / float(1 << 24)
