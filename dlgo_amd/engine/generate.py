"""The generation loop: requests in, token ids out.

The shape of computerex/dlgo's public loop (models/llm/generate.go:310-392): the
prompt goes through the model, then per step: stop if the sequence has reached
the context (:341), choose a token (:345), a stop token ends the sequence and is
not emitted (:347-359), else append it, report it (:367-372) and feed it back
(:385-386), for at most max_tokens tokens (:340).  Here many requests run
together: requests that fit (slots, cache pages for prompt plus max_tokens) form
a batch that starts together; their prompts are one step, then each live
sequence brings one token per step; a sequence that ends leaves the batch at
once and gives its slot back; when a batch is done the next one starts, in the
slots the last one freed.  Results come back in request order.

The loop decides with host data only and talks to the engine and the sampler
through four calls (open, close, step, choose), so its decisions can be tested
with stand-ins.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..sampling.options import GenerateConfig
from ..sampling.rng import resolve_seed, uniform
from ..sampling.sampler import RECENT
from .engine import Entry

PAGE = 64


@dataclass
class Result:
    tokens: List[int]
    finish_reason: str          # "stop" (a stop token), "length" (max_tokens), "context" (the context is full)
    prompt_tokens: int


@dataclass
class Stats:
    """What computerex/dlgo reports per call (models/llm/generate.go:192-200,275-282)."""
    prefill_ms: float = 0.0
    generate_ms: float = 0.0
    output_tokens: int = 0
    prompt_tokens: int = 0
    batches: int = 0
    steps: int = 0

    @property
    def tokens_per_sec(self) -> float:
        return self.output_tokens / (self.generate_ms / 1000.0) if self.generate_ms > 0 else 0.0


class GenerationError(ValueError):
    pass


@dataclass
class _Live:
    index: int
    slot: int
    config: GenerateConfig
    seed: int
    stop: frozenset
    pos: int
    tokens: List[int] = field(default_factory=list)


def plan_batch(prompt_lens: Sequence[int], max_new: Sequence[int], free_slots: int, free_pages: int, max_batch: int,
               max_ctx: int) -> int:
    """How many of the waiting requests (in order) start together: each needs a slot and, at worst,
    pages for min(prompt + max_new, context) tokens."""
    n, pages = 0, 0
    for p, m in zip(prompt_lens, max_new):
        need = (min(p + m, max_ctx) + PAGE - 1) // PAGE
        if n >= min(free_slots, max_batch) or pages + need > free_pages:
            break
        n += 1
        pages += need
    return n


def generate(engine, sampler, prompts: Sequence[Sequence[int]], configs: Sequence[GenerateConfig],
             default_stop: Sequence[int] = (), on_token: Optional[Callable[[int, int], None]] = None,
             max_batch: int = 64, sync: Optional[Callable[[], None]] = None):
    """Run every request; returns ([Result] in request order, Stats).

    engine: open(n) -> slots, close(slots), step(entries) -> logits rows, max_ctx, free_pages(), free_slots().
    sampler: choose(logits, sampler configs, uniforms, recent) -> token ids.
    on_token(request index, token id) is called once per emitted token.
    """
    if len(prompts) != len(configs):
        raise GenerationError("one configuration per prompt")
    for i, p in enumerate(prompts):
        if len(p) == 0:
            raise GenerationError(f"request {i}: empty prompt")
        if len(p) >= engine.max_ctx:
            raise GenerationError(f"request {i}: prompt too long: {len(p)} tokens (max {engine.max_ctx})")
    results: List[Optional[Result]] = [None] * len(prompts)
    stats = Stats()
    sync = sync or (lambda: None)
    waiting = list(range(len(prompts)))
    seeds = [resolve_seed(c.seed) for c in configs]
    while waiting:
        n = plan_batch([len(prompts[i]) for i in waiting], [configs[i].max_tokens for i in waiting],
                       engine.free_slots(), engine.free_pages(), max_batch, engine.max_ctx)
        if n == 0:
            i = waiting[0]
            raise GenerationError(f"request {i}: {len(prompts[i])} prompt tokens plus {configs[i].max_tokens} new ones do not fit the cache")
        batch, waiting = waiting[:n], waiting[n:]
        stats.batches += 1
        slots = engine.open(n)
        live: List[_Live] = []
        for i, s in zip(batch, slots):
            c = configs[i]
            stop = frozenset() if c.ignore_eos else frozenset(c.stop_tokens if c.stop_tokens is not None else default_stop)
            live.append(_Live(i, s, c, seeds[i], stop, len(prompts[i])))
        try:
            t0 = time.perf_counter()
            logits = engine.step([Entry(l.slot, list(prompts[l.index]), [len(prompts[l.index]) - 1]) for l in live])
            sync()
            t1 = time.perf_counter()
            stats.prefill_ms += (t1 - t0) * 1000.0
            stats.prompt_tokens += sum(len(prompts[l.index]) for l in live)
            stats.steps += 1
            while live:
                # sequences that may not go on leave before a token is chosen for them
                keep_rows = []
                for row, l in enumerate(live):
                    if len(l.tokens) >= l.config.max_tokens:
                        results[l.index] = Result(l.tokens, "length", len(prompts[l.index]))
                    elif l.pos >= engine.max_ctx - 1:
                        results[l.index] = Result(l.tokens, "context", len(prompts[l.index]))
                    else:
                        keep_rows.append(row)
                        continue
                    engine.close([l.slot])
                if not keep_rows:
                    live = []
                    break
                if len(keep_rows) != len(live):
                    logits = logits[keep_rows] if hasattr(logits, "__getitem__") else logits
                    live = [live[r] for r in keep_rows]
                chosen = sampler.choose(logits, [l.config.sampler for l in live],
                                        [uniform(l.seed, l.index, len(l.tokens)) for l in live],
                                        [l.tokens[-RECENT:] for l in live])
                nxt: List[_Live] = []
                for l, tok in zip(live, chosen):
                    tok = int(tok)
                    if tok in l.stop:
                        results[l.index] = Result(l.tokens, "stop", len(prompts[l.index]))
                        engine.close([l.slot])
                        continue
                    l.tokens.append(tok)
                    stats.output_tokens += 1
                    if on_token is not None:
                        on_token(l.index, tok)
                    if len(l.tokens) >= l.config.max_tokens:
                        results[l.index] = Result(l.tokens, "length", len(prompts[l.index]))
                        engine.close([l.slot])
                        continue
                    nxt.append(l)
                live = nxt
                if not live:
                    break
                logits = engine.step([Entry(l.slot, [l.tokens[-1]], [0]) for l in live])
                stats.steps += 1
                for l in live:
                    l.pos += 1
            sync()
            stats.generate_ms += (time.perf_counter() - t1) * 1000.0
        except BaseException:
            for l in live:
                if results[l.index] is None:
                    try:
                        engine.close([l.slot])
                    except Exception:
                        pass
            raise
    return results, stats
