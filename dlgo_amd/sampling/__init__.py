from .options import (GenerateConfig, Option, SamplerConfig, apply_options, with_greedy, with_ignore_eos,
                      with_max_tokens, with_min_p, with_repetition_penalty, with_seed, with_stop_tokens,
                      with_temperature, with_top_k, with_top_p)
from .rng import resolve_seed, uniform

__all__ = ["GenerateConfig", "Option", "SamplerConfig", "apply_options", "with_greedy", "with_ignore_eos",
           "with_max_tokens", "with_min_p", "with_repetition_penalty", "with_seed", "with_stop_tokens",
           "with_temperature", "with_top_k", "with_top_p", "resolve_seed", "uniform"]
from .sampler import RECENT, Sampler  # noqa: E402

__all__ += ["RECENT", "Sampler"]
