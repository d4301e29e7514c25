"""Sampling and generation options, with computerex/dlgo's names, meanings and
defaults: SamplerConfig (ops/sampling.go:10-27: temperature 0.7, top-k 40, top-p
0.9, min-p 0, repetition penalty 1.1), GenerateConfig (models/llm/generate.go:17-31:
256 tokens, seed -1 = from the clock), and the functional options of dlgo.go:209-248."""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Callable, Optional, Sequence, Tuple


@dataclass
class SamplerConfig:
    temperature: float = 0.7        # 0 = greedy
    top_k: int = 40                 # 0 = off
    top_p: float = 0.9              # 1.0 = off
    min_p: float = 0.0              # 0 = off
    repetition_penalty: float = 1.1  # 1.0 = off

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0


@dataclass
class GenerateConfig:
    max_tokens: int = 256
    sampler: SamplerConfig = field(default_factory=SamplerConfig)
    seed: int = -1                               # < 0: seeded from the clock
    stop_tokens: Optional[Tuple[int, ...]] = None   # None: the model's own (eos ids of its configuration)
    ignore_eos: bool = False                     # benchmarks: never stop on a token


Option = Callable[[GenerateConfig], None]


def with_max_tokens(n: int) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.max_tokens = int(n)
    return opt


def with_temperature(t: float) -> Option:
    """0 = greedy, 0.7 = creative (dlgo.go:218-221)."""
    def opt(c: GenerateConfig) -> None:
        c.sampler.temperature = float(t)
    return opt


def with_top_k(k: int) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.sampler.top_k = int(k)
    return opt


def with_top_p(p: float) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.sampler.top_p = float(p)
    return opt


def with_min_p(p: float) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.sampler.min_p = float(p)
    return opt


def with_repetition_penalty(p: float) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.sampler.repetition_penalty = float(p)
    return opt


def with_seed(seed: int) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.seed = int(seed)
    return opt


def with_greedy() -> Option:
    """Argmax decoding: temperature 0 (dlgo.go:238-240)."""
    def opt(c: GenerateConfig) -> None:
        c.sampler.temperature = 0.0
    return opt


def with_stop_tokens(tokens: Sequence[int]) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.stop_tokens = tuple(int(t) for t in tokens)
    return opt


def with_ignore_eos(on: bool = True) -> Option:
    def opt(c: GenerateConfig) -> None:
        c.ignore_eos = bool(on)
    return opt


def apply_options(opts: Sequence[Option], base: Optional[GenerateConfig] = None) -> GenerateConfig:
    """Options over the defaults (dlgo.go:242-248)."""
    cfg = copy.deepcopy(base) if base is not None else GenerateConfig()
    for o in opts:
        o(cfg)
    if cfg.max_tokens < 0:
        raise ValueError("max_tokens must be >= 0")
    if cfg.sampler.temperature < 0:
        raise ValueError("temperature must be >= 0")
    return cfg
