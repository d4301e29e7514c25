"""The Python entry point, in the manner of computerex/dlgo's dlgo.go: LoadLLM
(:37) -> load_llm, (*LLM).Generate (:51) -> LLM.generate, GenerateStream (:79) ->
LLM.generate_stream, Benchmark (:93) -> LLM.benchmark, ModelInfo (:117) ->
LLM.model_info, and the With* options (:209-240).  Token ids go in and come out;
tokenizers and chat templates are not part of this library.
"""
from __future__ import annotations

import operator
from dataclasses import dataclass
from typing import Callable, List, Mapping, Optional, Sequence, Union

import torch

from .cache import PAGE, tokens_that_fit
from .config import ModelConfig, build_model, config_from_dict, load_config
from .engine.engine import Engine, EngineError, recordings_bytes, run_dtype
from .weights import load_state, load_weights, random_tensors
from .engine.generate import GenerationError, Result, Stats, generate
from .sampling import GenerateConfig, Option, Sampler, apply_options

Prompt = Sequence[int]


@dataclass
class GenerateResult:
    """dlgo.go:187-207: the output with the timings of the call."""
    tokens: List[int]
    finish_reason: str
    tokens_per_sec: float
    prefill_ms: float
    generate_ms: float
    output_tokens: int
    prompt_tokens: int

    def __str__(self) -> str:
        return (f"{self.tokens_per_sec:.1f} tok/s | prefill: {self.prefill_ms:.0f}ms | gen: {self.generate_ms:.0f}ms | "
                f"{self.output_tokens} tokens | {self.finish_reason}")


@dataclass
class BenchmarkResult:
    """dlgo.go:152-168, with the time of every step beside the totals (step_ms[0] is the prompt step)."""
    tokens: List[int]
    tokens_per_sec: float
    prefill_ms: float
    generate_ms: float
    total_ms: float
    prompt_tokens: int
    output_tokens: int
    architecture: str
    step_ms: List[float]


def _is_id(x) -> bool:
    """An integer of any kind (Python's, numpy's, an element of an integer tensor), not a float and not a sequence."""
    try:
        operator.index(x)
        return True
    except TypeError:
        return False


def _ids(prompt, i: int) -> List[int]:
    try:
        return [operator.index(t) for t in prompt]
    except TypeError:
        raise GenerationError(f"request {i}: a prompt is a sequence of integer token ids") from None


class LLM:
    def __init__(self, engine: Engine, max_batch: int = 64):
        self.engine = engine
        self.config: ModelConfig = engine.model.config
        self.max_seq_len = engine.max_ctx
        self.max_batch = max_batch
        self.sampler = Sampler(engine.vocab, engine.device, max_rows=max_batch)
        self.stop_tokens = tuple(self.config.stop_tokens())

    def _run(self, prompts: Sequence[Prompt], opts: Sequence[Option], on_token=None):
        prompts = [_ids(p, i) for i, p in enumerate(prompts)]
        cfg = apply_options(opts)
        results, stats = generate(self.engine, self.sampler, prompts, [cfg] * len(prompts), self.stop_tokens, on_token,
                                  self.max_batch, sync=torch.cuda.synchronize)
        return results, stats

    @staticmethod
    def _wrap(r: Result, s: Stats) -> GenerateResult:
        return GenerateResult(r.tokens, r.finish_reason, s.tokens_per_sec, s.prefill_ms, s.generate_ms, len(r.tokens),
                              r.prompt_tokens)

    def generate(self, prompt: Union[Prompt, Sequence[Prompt]], *opts: Option):
        """One prompt (a list of token ids) -> GenerateResult; a list of prompts -> a list of them, run as
        batches of unequal lengths."""
        many = len(prompt) > 0 and not _is_id(prompt[0])
        prompts = list(prompt) if many else [prompt]
        results, stats = self._run(prompts, opts)
        out = [self._wrap(r, stats) for r in results]
        return out if many else out[0]

    def generate_stream(self, prompt: Prompt, on_token: Callable[[int], None], *opts: Option) -> GenerateResult:
        """on_token(token id) is called for every token as it is generated (dlgo.go:79-90)."""
        results, stats = self._run([prompt], opts, on_token=lambda i, t: on_token(t))
        return self._wrap(results[0], stats)

    def benchmark(self, prompt: Prompt, *opts: Option) -> "BenchmarkResult":
        """A run with separate prefill and generation timings, the whole call's time and the time of every step
        (dlgo.go:93-114; models/llm/generate.go:227-229,275-282)."""
        import time
        t0 = time.perf_counter()
        results, stats = self._run([prompt], opts)
        total_ms = (time.perf_counter() - t0) * 1000.0
        r = results[0]
        return BenchmarkResult(r.tokens, stats.tokens_per_sec, stats.prefill_ms, stats.generate_ms, total_ms, r.prompt_tokens,
                               len(r.tokens), self.config.architecture, list(stats.step_ms))

    def model_info(self) -> str:
        """dlgo.go:170-185."""
        return " | ".join([self.config.architecture, *self.config.describe(), f"ctx {self.max_seq_len}",
                           str(self.engine.dtype).replace('torch.', '')])


def load_llm(model: Union[str, ModelConfig, Mapping], max_seq_len: int = 0, dtype: str = "bfloat16", device: str = "cuda:0",
             max_batch: int = 64, max_tokens: Optional[int] = None, random_seed: Optional[int] = None,
             random_std: Optional[float] = None, **engine_options) -> LLM:
    """Load a model folder (config.json, model.safetensors), as dlgo.go:37-47 loads a file.  With `random_seed` the
    weights are drawn for that seed instead of read, and `model` may then also be a config.json file, its contents as
    a mapping, or a configuration object: nothing is written (a folder given with a seed lends its config.json only).
    max_seq_len <= 0 or beyond the model's context means the model's context (models/llm/generate.go:56-58).  The
    cache is sized for `max_tokens` tokens over all live sequences; by default for max_batch sequences of max_seq_len,
    or for as many tokens as the device's free memory holds once the weights are loaded (a fifth of it stays free,
    and room for the recordings of steps), if that is less."""
    if isinstance(model, ModelConfig):
        config = model
    elif isinstance(model, Mapping):
        config = config_from_dict(model)
    else:
        config = load_config(model)
    if random_seed is None and not isinstance(model, str):
        raise EngineError("load_llm: a configuration without a model folder needs random_seed (there are no weights to read)")
    limit = config.context_length()
    ctx = max_seq_len if max_seq_len > 0 and (limit is None or max_seq_len <= limit) else limit
    if not torch.cuda.is_available():
        raise EngineError("no HIP device: dlgo_amd runs on an AMD GPU only and has no CPU path")
    rd = run_dtype(dtype)
    built = build_model(config)
    if random_seed is None:
        load_weights(built, model, device, rd)
    else:
        tensors = random_tensors(config, random_seed, rd, random_std, device=device)
        load_state(built, tensors, device, rd, where="random weights")
        del tensors
    if max_tokens is None:
        free, _ = torch.cuda.mem_get_info(torch.device(device))
        fit = tokens_that_fit(built.unit_needs, rd, free, recordings_bytes(built.vocab, max_batch, **engine_options))
        if fit < PAGE:
            raise EngineError(f"no device memory left for a cache ({free >> 20} MiB free after the weights)")
        max_tokens = fit if ctx is None else min(max_batch * ctx, fit)
    engine = Engine(built, rd, device, max_tokens=max_tokens, max_ctx=ctx, **engine_options)
    return LLM(engine, max_batch)
