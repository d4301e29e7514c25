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
through a handful of calls, so its decisions can be tested with stand-ins:

    engine:  open(n) -> slots, close(slots), step(entries) -> logits rows (the prompts),
             decode(slots, ids) -> logits rows (one token each; ids as the sampler left them on the device),
             max_ctx, free_slots(), free_pages() and page_demand(n_tokens) (per storage group of the cache)
    sampler: start(keys), choose_async(logits, configs, uniforms, keys=) -> (ids on the device, wait() -> ids on the host)

The loop runs one step ahead of the host: the step that feeds the tokens just
chosen is queued before those tokens reach the host, so the GPU does not wait
for the host's bookkeeping.  Whether a sequence goes on after a token is then
known one step late: a sequence that turns out to have stopped has been given
one step too many, whose result is dropped and whose slot is given back as
before.  The sampler keeps each request's recent tokens itself (by key: the
request's slot), so the repetition penalty does not need them back first.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..sampling.options import GenerateConfig
from ..sampling.rng import resolve_seed, uniform
from .engine import Entry

@dataclass
class Result:
    tokens: List[int]
    finish_reason: str          # "stop" (a stop token), "length" (max_tokens), "context" (the context is full)
    prompt_tokens: int


@dataclass
class Stats:
    """What computerex/dlgo reports per call (models/llm/generate.go:192-200,227-229,275-282), and the time of every
    step: step_ms[0] of a batch is its prompt step, the others are the times from one step's tokens reaching the
    host to the next step's (the loop runs a step ahead, so that is what a step costs)."""
    prefill_ms: float = 0.0
    generate_ms: float = 0.0
    output_tokens: int = 0
    prompt_tokens: int = 0
    batches: int = 0
    steps: int = 0
    step_ms: List[float] = field(default_factory=list)

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


def plan_batch(prompt_lens: Sequence[int], max_new: Sequence[int], free_slots: int, free_pages: Sequence[int], max_batch: int,
               max_ctx: int, page_demand: Callable[[int], Sequence[int]]) -> int:
    """How many of the waiting requests (in order) start together: each needs a slot and, at worst, in every storage
    group of the cache the pages that page_demand gives for min(prompt + max_new, context) tokens."""
    n = 0
    used = [0] * len(free_pages)
    for p, m in zip(prompt_lens, max_new):
        need = page_demand(min(p + m, max_ctx))
        if n >= min(free_slots, max_batch) or any(u + d > f for u, d, f in zip(used, need, free_pages)):
            break
        n += 1
        used = [u + d for u, d in zip(used, need)]
    return n


def _take(engine, x, rows):
    """x[rows] for row numbers the host knows: the engine's own row copy where it has one (the rows stay on the
    device and nothing waits), plain indexing for a stand-in."""
    take = getattr(engine, "take_rows", None)
    return take(x, rows) if take is not None else x[rows]


def _decode_batch(engine, sampler, live, logits, prompts, results, stats, on_token) -> None:
    """The decode loop of one batch, one step ahead of the host (see the module's text).  `logits` has one row per
    entry of `live`, in order."""
    def finish(l, reason):
        results[l.index] = Result(l.tokens, reason, len(prompts[l.index]))
        engine.close([l.slot])
        l.slot = -1

    last = time.perf_counter()
    while live:
        # before a token is chosen: who may not go on at all
        keep = []
        for row, l in enumerate(live):
            if len(l.tokens) >= l.config.max_tokens:
                finish(l, "length")
            elif l.pos >= engine.max_ctx - 1:
                finish(l, "context")
            else:
                keep.append(row)
        if not keep:
            return
        if len(keep) != len(live):
            logits = _take(engine, logits, keep)
            live = [live[r] for r in keep]
        ids, wait = sampler.choose_async(logits, [l.config.sampler for l in live],
                                         [uniform(l.seed, l.index, len(l.tokens)) for l in live], keys=[l.slot for l in live])
        # queue the next step for every sequence that wants another token after this one, before knowing the ids
        fed = [row for row, l in enumerate(live) if len(l.tokens) + 1 < l.config.max_tokens and l.pos + 1 < engine.max_ctx - 1]
        next_logits = None
        if fed:
            next_logits = engine.decode([live[r].slot for r in fed], ids if len(fed) == len(live) else _take(engine, ids, fed))
            stats.steps += 1
        chosen = wait()
        now = time.perf_counter()
        stats.step_ms.append((now - last) * 1000.0)
        last = now
        still = []
        for row, (l, tok) in enumerate(zip(live, chosen)):
            tok = int(tok)
            if tok in l.stop:
                finish(l, "stop")         # if it was fed, that step's row is dropped
                continue
            l.tokens.append(tok)
            l.pos += 1
            stats.output_tokens += 1
            if on_token is not None:
                on_token(l.index, tok)
            if len(l.tokens) >= l.config.max_tokens:
                finish(l, "length")
            elif l.pos >= engine.max_ctx - 1:
                finish(l, "context")
            else:
                still.append(row)
        if not still:
            return
        rows = [fed.index(r) for r in still]          # every row in `still` was fed
        logits = next_logits if len(rows) == len(fed) else _take(engine, next_logits, rows)
        live = [live[r] for r in still]


def generate(engine, sampler, prompts: Sequence[Sequence[int]], configs: Sequence[GenerateConfig],
             default_stop: Sequence[int] = (), on_token: Optional[Callable[[int, int], None]] = None,
             max_batch: int = 64, sync: Optional[Callable[[], None]] = None):
    """Run every request; returns ([Result] in request order, Stats).  on_token(request index, token id) is called once
    per emitted token; sync() waits for the device (for the timings)."""
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
                       engine.free_slots(), engine.free_pages(), max_batch, engine.max_ctx, engine.page_demand)
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
            stats.step_ms.append((t1 - t0) * 1000.0)
            stats.prompt_tokens += sum(len(prompts[l.index]) for l in live)
            stats.steps += 1
            sampler.start([l.slot for l in live])
            _decode_batch(engine, sampler, live, logits, prompts, results, stats, on_token)
            sync()
            stats.generate_ms += (time.perf_counter() - t1) * 1000.0
        except BaseException:
            for l in live:
                if results[l.index] is None and l.slot >= 0:
                    try:
                        engine.close([l.slot])
                    except Exception:
                        pass
            raise
    return results, stats
