"""dlgo_amd: a small language-model library for one AMD MI355X (gfx950): typed
configuration, weights by name, layers made of parts, a paged cache, one step
function, a generation loop, samplers, and hand-written HIP kernels beneath."""
from .sampling.options import (GenerateConfig, SamplerConfig, with_greedy, with_ignore_eos, with_max_tokens, with_min_p,
                               with_repetition_penalty, with_seed, with_stop_tokens, with_temperature, with_top_k,
                               with_top_p)

# computerex/dlgo's spellings (dlgo.go:213-240)
WithMaxTokens, WithTemperature, WithTopK, WithTopP = with_max_tokens, with_temperature, with_top_k, with_top_p
WithSeed, WithGreedy = with_seed, with_greedy


def load_llm(*args, **kwargs):
    from .api import load_llm as _load
    return _load(*args, **kwargs)


LoadLLM = load_llm

__all__ = ["GenerateConfig", "SamplerConfig", "load_llm", "LoadLLM", "with_greedy", "with_ignore_eos", "with_max_tokens",
           "with_min_p", "with_repetition_penalty", "with_seed", "with_stop_tokens", "with_temperature", "with_top_k",
           "with_top_p", "WithMaxTokens", "WithTemperature", "WithTopK", "WithTopP", "WithSeed", "WithGreedy"]
