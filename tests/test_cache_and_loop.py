"""The cache's bookkeeping (no slot or page lost, held twice or freed twice) and the generation
loop's decisions, with stand-ins for the engine and the sampler; no GPU."""
import random

import numpy as np
import pytest
import torch

from dlgo_amd.cache import PAGE, Cache, CacheError, OutOfPages, PagePool
from dlgo_amd.engine.generate import GenerationError, generate, plan_batch
from dlgo_amd.parts import CacheNeed
from dlgo_amd.sampling import GenerateConfig, SamplerConfig, apply_options, uniform, with_greedy, with_max_tokens, \
    with_seed, with_temperature, with_top_k, with_top_p

KV = [CacheNeed(kind="kv", kv_heads=2, head_dim=16)]


def make_cache(n_units=2, max_tokens=8 * PAGE, max_ctx=4 * PAGE, needs=None, **kw):
    return Cache([needs or KV for _ in range(n_units)], max_tokens, max_ctx, torch.float32, "cpu", **kw)


def test_page_pool():
    pool = PagePool(4)
    a = pool.take(3)
    assert sorted(a) == [0, 1, 2] and pool.n_free == 1
    with pytest.raises(OutOfPages):
        pool.take(2)
    pool.give(a[:1])
    with pytest.raises(CacheError):
        pool.give(a[:1])              # freed twice
    with pytest.raises(CacheError):
        pool.give([7])                # not a page of this pool
    assert pool.n_free == 2


def test_slots_and_pages_round_trip():
    c = make_cache()
    assert c.n_pages == 8 and c.max_pages_per_seq == 4 and len(c.groups) == 1      # both units share one group
    g = c.groups[0]
    assert g.page_stride == 2 * g.unit_elems and g.storage.numel() == 8 * g.page_stride
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([(a, 70), (b, 1)])
    assert len(c.held_pages(a)) == 2 and len(c.held_pages(b)) == 1 and g.pool.n_free == 5
    c.advance(a, 70)
    c.advance(b, 1)
    assert c.length(a) == 70
    c.reserve([(a, 71), (b, 2)])                          # nothing new needed
    assert g.pool.n_free == 5
    c.reserve([(a, 129)])
    assert len(c.held_pages(a)) == 3
    assert (g.table_host[a, :3] >= 0).all() and g.table_host[a, 3] == -1
    c.check_consistent()
    c.free_slot(a)
    assert g.pool.n_free == 7 and (g.table_host[a] == -1).all()
    with pytest.raises(CacheError):
        c.free_slot(a)                                    # freed twice
    with pytest.raises(CacheError):
        c.length(a)
    c.sync_tables()
    assert torch.equal(g.table, torch.from_numpy(g.table_host))
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0                  # the slot is used again, empty
    c.check_consistent()


def test_limits_are_errors_before_anything_changes():
    c = make_cache(max_tokens=3 * PAGE, max_ctx=2 * PAGE)
    s = [c.alloc_slot() for _ in range(3)]
    with pytest.raises(CacheError, match="no free slot"):
        c.alloc_slot()
    assert "context" in c.can_reserve([(s[0], 2 * PAGE + 1)])
    c.reserve([(s[0], 2 * PAGE)])
    before = c.groups[0].pool.n_free
    with pytest.raises(OutOfPages):
        c.reserve([(s[1], 1), (s[2], 65)])
    assert c.groups[0].pool.n_free == before and not c.held_pages(s[1])
    c.check_consistent()


def test_groups_by_need_and_window_release():
    needs = [[CacheNeed("kv", 2, 16)], [CacheNeed("kv", 2, 16, window=100)], [CacheNeed("kv", 1, 32)],
             [CacheNeed("kv", 2, 16), CacheNeed("state", state_shape=(3, 4))], [CacheNeed("none")]]
    c = Cache(needs, 64 * PAGE, 32 * PAGE, torch.float32, "cpu", max_slots=4, max_step_tokens=128)
    assert len(c.groups) == 3
    assert [c.unit_group.get(u) for u in range(5)] == [(0, 0), (1, 0), (2, 0), (0, 1), None]
    windowed = c.groups[1]
    assert windowed.pool.n_pages == 4 * ((100 + 128 + 63) // 64 + 1) < c.groups[0].pool.n_pages      # storage of its own, smaller
    assert c.state_of(3).shape == (4, 3, 4)
    s = c.alloc_slot()
    total = 0
    for step in [128, 128, 100, 1, 1, 64, 128]:
        c.reserve([(s, total + step)])
        c.advance(s, step)
        total += step
        held = c.held_pages(s, 1)
        first_needed = max(0, total - 100 + 1) // PAGE
        assert min(held) == first_needed and max(held) == (total - 1) // PAGE       # a window of pages, no more
        assert len(c.held_pages(s, 0)) == (total + PAGE - 1) // PAGE                # the full group keeps everything
        c.check_consistent()
    kv = c.kv_view(1)
    assert kv.window == 100 and kv.page_table is windowed.table
    c.free_slot(s)
    assert all(g.pool.n_free == g.pool.n_pages for g in c.groups)


def test_copy_of_a_slot_has_pages_of_its_own():
    """memory/kvcache.go:38-55 (Clone): a deep copy up to a position.  Here: pages of its own with the same content, the
    same length, the state as it is; nothing shared, so either can go on or be given back without the other noticing."""
    needs = [[CacheNeed("kv", 2, 16)], [CacheNeed("kv", 2, 16, window=100)], [CacheNeed("kv", 2, 16), CacheNeed("state", state_shape=(3,))]]
    c = Cache(needs, 64 * PAGE, 32 * PAGE, torch.float32, "cpu", max_slots=4, max_step_tokens=128)
    a = c.alloc_slot()
    total = 0
    for step in [128, 100, 1, 64]:
        c.reserve([(a, total + step)])
        c.advance(a, step)
        total += step
    for g in c.groups:                                   # every page of the pool tells its own number
        g.storage.view(g.pool.n_pages, g.page_stride)[:] = torch.arange(g.pool.n_pages, dtype=torch.float32)[:, None]
    c.state_of(2)[a] = torch.tensor([1.0, 2.0, 3.0])
    b = c.copy_slot(a)
    c.check_consistent()
    assert b != a and c.length(b) == total == 293
    for gi, g in enumerate(c.groups):
        pa, pb = c.held_pages(a, gi), c.held_pages(b, gi)
        assert sorted(pa) == sorted(pb) and not set(pa.values()) & set(pb.values())
        by_page = g.storage.view(g.pool.n_pages, g.page_stride)
        for i in pa:
            assert torch.equal(by_page[pb[i]], by_page[pa[i]]) and by_page[pb[i]][0] == pa[i]
        assert (g.table_host[b, sorted(pb)] == [pb[i] for i in sorted(pb)]).all()
    assert torch.equal(c.state_of(2)[b], torch.tensor([1.0, 2.0, 3.0]))
    # the two go their own ways
    c.reserve([(b, total + 70)])
    c.advance(b, 70)
    assert c.length(a) == total and c.length(b) == total + 70
    c.free_slot(a)
    c.check_consistent()
    assert c.length(b) == total + 70 and len(c.held_pages(b, 0)) == (total + 70 + PAGE - 1) // PAGE
    c.free_slot(b)
    assert all(g.pool.n_free == g.pool.n_pages for g in c.groups)
    # an earlier length: only where nothing depends on what came after it
    plain = make_cache(n_units=2, max_tokens=8 * PAGE, max_ctx=4 * PAGE)
    s = plain.alloc_slot()
    plain.reserve([(s, 150)])
    plain.advance(s, 150)
    t = plain.copy_slot(s, 70)
    assert plain.length(t) == 70 and sorted(plain.held_pages(t)) == [0, 1]
    with pytest.raises(CacheError, match="holds 150 tokens"):
        plain.copy_slot(s, 151)
    u = c.alloc_slot()
    c.reserve([(u, 10)])
    c.advance(u, 10)
    with pytest.raises(CacheError, match="state"):
        c.copy_slot(u, 5)
    windowed = Cache([[CacheNeed("kv", 2, 16, window=100)]], 64 * PAGE, 32 * PAGE, torch.float32, "cpu", max_slots=4, max_step_tokens=128)
    w = windowed.alloc_slot()
    for step in [128, 128, 128]:
        windowed.reserve([(w, windowed.length(w) + step)])
        windowed.advance(w, step)
    with pytest.raises(CacheError, match="no longer holds"):
        windowed.copy_slot(w, 100)
    # no room: nothing changes
    full = make_cache(n_units=1, max_tokens=4 * PAGE, max_ctx=4 * PAGE, max_slots=3)
    f = full.alloc_slot()
    full.reserve([(f, 3 * PAGE)])
    full.advance(f, 3 * PAGE)
    with pytest.raises(CacheError, match="cache full"):
        full.copy_slot(f)
    full.check_consistent()
    assert full.live_slots() == [f] and full.groups[0].pool.n_free == 1


def test_state_is_zeroed_when_a_slot_is_handed_out():
    c = Cache([[CacheNeed("state", state_shape=(5,), state_dtype=torch.float32)]], PAGE, PAGE, torch.float32, "cpu", max_slots=2)
    s = c.alloc_slot()
    c.state_of(0)[s] = 7.0
    c.free_slot(s)
    t = c.alloc_slot()
    assert t == s and torch.equal(c.state_of(0)[t], torch.zeros(5))


def test_workspace_buffers_keep_their_place():
    """A step's scratch rows: a buffer per (name, width, type) that never moves, so that a recorded step can be
    replayed; the view made for one layer serves the next one that asks for the same rows, and other rows or another
    width get views of their own."""
    from dlgo_amd.engine.context import Workspace
    ws = Workspace(torch.device("cpu"), 16)
    a = ws.get("rows", (5, 8), torch.float32)
    assert tuple(a.shape) == (5, 8) and ws.get("rows", (5, 8), torch.float32) is a
    b = ws.get("rows", (7, 8), torch.float32)
    assert tuple(b.shape) == (7, 8) and b.data_ptr() == a.data_ptr()          # more rows of the same buffer
    c = ws.get("rows", (5, 4, 2), torch.float32)
    assert tuple(c.shape) == (5, 4, 2) and c.data_ptr() == a.data_ptr()       # the same width, seen as 4 x 2
    d = ws.get("rows", (5, 6), torch.float32)
    e = ws.get("rows", (5, 8), torch.bfloat16)
    assert len({a.data_ptr(), d.data_ptr(), e.data_ptr()}) == 3              # another width, another type: other buffers
    a.fill_(3.0)
    assert float(ws.get("rows", (5, 8), torch.float32)[4, 7]) == 3.0          # and the first one is still where it was
    assert tuple(ws.get("flags", (9,), torch.int32).shape) == (9,)
    with pytest.raises(RuntimeError, match="room for 16"):
        ws.get("rows", (17, 8), torch.float32)
    f1 = ws.flat("runs", 100, torch.float32)
    assert ws.flat("runs", 50, torch.float32) is f1 and ws.flat("runs", 200, torch.float32).numel() >= 200
    assert ws.bytes() > 0


def test_random_traffic_keeps_the_books():
    rng = random.Random(0)
    c = make_cache(n_units=3, max_tokens=40 * PAGE, max_ctx=10 * PAGE, max_slots=6,
                   needs=[CacheNeed("kv", 2, 16), ])
    live = {}
    for _ in range(600):
        r = rng.random()
        if r < 0.25 and c.n_free_slots:
            live[c.alloc_slot()] = 0
        elif r < 0.4 and live:
            s = rng.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 5, 64, 130])
            if live[s] + n <= c.max_ctx and c.can_reserve([(s, live[s] + n)]) is None:
                c.reserve([(s, live[s] + n)])
                c.advance(s, n)
                live[s] += n
        c.check_consistent()
        assert sorted(live) == c.live_slots()
        assert all(c.length(s) == n for s, n in live.items())
        held = sum((n + PAGE - 1) // PAGE for n in live.values())
        assert c.groups[0].pool.n_free == 40 - held


def test_a_cache_of_windowed_groups_only_is_counted_too():
    """No full group to run out first: the windowed pool itself is what a step is checked against, before anything is
    taken, and what the loop plans with."""
    need = [CacheNeed(kind="kv", kv_heads=2, head_dim=16, window=100)]
    c = Cache([need], max_tokens=8 * PAGE, max_ctx=8 * PAGE, dtype=torch.float32, device="cpu", max_slots=3, max_step_tokens=64)
    assert c.groups[0].pool.n_pages == 8 and c.groups[0].pages_per_seq == 4       # window + a step's piece, in pages, + 1
    assert c.page_demand(500) == (4,) and c.page_demand(70) == (2,) and c.free_pages() == (8,)
    assert plan_batch([400, 400, 400], [50, 50, 50], 3, c.free_pages(), 64, c.max_ctx, c.page_demand) == 2
    slots = [c.alloc_slot() for _ in range(3)]

    def grow(slot, total):                       # a long prompt, in pieces of a step's size
        while c.length(slot) < total:
            n = min(64, total - c.length(slot))
            assert c.can_reserve([(slot, c.length(slot) + n)]) is None
            c.reserve([(slot, c.length(slot) + n)])
            c.advance(slot, n)
            c.check_consistent()
            assert len(c.held_pages(slot)) <= 4
    grow(slots[0], 400)
    grow(slots[1], 400)
    held = len(c.held_pages(slots[0])) + len(c.held_pages(slots[1]))
    assert c.free_pages() == (8 - held,)
    # a whole long prompt is judged by what it holds at worst, not by its length
    assert c.can_reserve([(slots[0], 512)]) is None
    # the third sequence does not fit beside them: the check says so, and nothing was taken
    free = c.free_pages()
    why = c.can_reserve([(slots[2], 64 * (free[0] + 1))])
    assert why is not None and "cache full" in why
    with pytest.raises(OutOfPages):
        c.reserve([(slots[2], 64 * (free[0] + 1))])
    assert c.free_pages() == free and not c.held_pages(slots[2])
    c.check_consistent()
    c.free_slot(slots[0])
    grow(slots[2], 200)
    for s in slots[1:]:
        c.free_slot(s)
    assert c.free_pages() == (8,)
    c.check_consistent()


# -- the generation loop -------------------------------------------------------------
class FakeEngine:
    """Slots and pages like the real one; 'logits' are rows (slot, tokens held) that the sampler decides on.  Like the
    real one it takes the prompts through step() and single tokens through decode(), whose ids are whatever the
    sampler left 'on the device' (here: an array whose values the loop has not looked at yet)."""

    def __init__(self, max_ctx=64, slots=3, pages=6):
        self.max_ctx, self._slots, self._pages = max_ctx, slots, pages
        self.free = list(range(slots))
        self.held = {}
        self.steps = []
        self.closed = []

    def free_slots(self):
        return len(self.free)

    def free_pages(self):
        return (self._pages - sum((n + PAGE - 1) // PAGE for n in self.held.values()),)

    def page_demand(self, n_tokens):
        return ((n_tokens + PAGE - 1) // PAGE,)

    def open(self, n):
        out = [self.free.pop(0) for _ in range(n)]
        for s in out:
            self.held[s] = 0
        return out

    def close(self, slots):
        for s in slots:
            assert s in self.held, "slot closed twice"
            del self.held[s]
            self.free.append(s)
            self.closed.append(s)

    def _run(self, rows):
        assert len({slot for slot, _, _ in rows}) == len(rows)
        for slot, tokens, _ in rows:
            assert slot in self.held, "a step for a slot that was given back"
            self.held[slot] += len(tokens)
            assert self.held[slot] <= self.max_ctx
        assert self.free_pages()[0] >= 0
        self.steps.append(rows)
        return np.array([(slot, self.held[slot]) for slot, _, _ in rows])

    def step(self, entries):
        return self._run([(e.slot, list(e.tokens), list(e.want)) for e in entries])

    def decode(self, slots, ids):
        assert len(slots) == len(ids)
        return self._run([(int(s), [int(t)], [0]) for s, t in zip(slots, ids)])


class ScriptSampler:
    """Token = 100 + length of the sequence so far, or a scripted stop.  It keeps each key's recent tokens itself, as the
    real one does on the device."""

    def __init__(self, stop_at=None):
        self.stop_at = stop_at or {}
        self.calls = []
        self.recent = {}
        self.waited = 0

    def start(self, keys):
        for k in keys:
            self.recent[k] = []

    def choose_async(self, logits, configs, uniforms, recent=None, keys=None):
        assert recent is None and len(keys) == len(logits) == len(configs) == len(uniforms)
        assert all(int(slot) == k for (slot, _), k in zip(logits, keys)), "rows and keys out of step"
        self.calls.append(([tuple(r) for r in logits], list(uniforms), [list(self.recent[k]) for k in keys]))
        ids = np.array([self.stop_at.get((int(slot), int(n)), 100 + int(n)) for slot, n in logits])
        for k, t in zip(keys, ids):
            self.recent[k] = (self.recent[k] + [int(t)])[-64:]

        def wait():
            self.waited += 1
            return ids.tolist()
        return ids, wait


def one_group(n):
    return ((n + PAGE - 1) // PAGE,)


def test_plan_batch():
    assert plan_batch([5, 9, 1], [8, 8, 8], 3, (6,), max_batch=64, max_ctx=4096, page_demand=one_group) == 3
    assert plan_batch([5, 9, 1], [8, 8, 8], 2, (6,), max_batch=64, max_ctx=4096, page_demand=one_group) == 2
    assert plan_batch([60, 60, 60], [8, 8, 8], 3, (5,), max_batch=64, max_ctx=4096, page_demand=one_group) == 2
    assert plan_batch([60, 60], [1000, 8], 3, (2,), max_batch=64, max_ctx=64, page_demand=one_group) == 2      # capped by the context
    assert plan_batch([200], [8], 3, (2,), max_batch=64, max_ctx=4096, page_demand=one_group) == 0
    assert plan_batch([1] * 9, [1] * 9, 9, (9,), max_batch=4, max_ctx=64, page_demand=one_group) == 4
    # every storage group of the cache counts: a second, windowed group that allows two pages a sequence
    two = lambda n: ((n + PAGE - 1) // PAGE, min((n + PAGE - 1) // PAGE, 2))
    assert plan_batch([300, 300, 300], [8, 8, 8], 3, (100, 5), max_batch=64, max_ctx=4096, page_demand=two) == 2
    # and a model that keeps no keys or values at all is limited by its slots only
    assert plan_batch([300, 300, 300], [8, 8, 8], 2, (), max_batch=64, max_ctx=4096, page_demand=lambda n: ()) == 2


def test_loop_unequal_batch_early_finishers_and_slot_reuse():
    eng, samp = FakeEngine(), ScriptSampler()
    cfgs = [GenerateConfig(max_tokens=n, sampler=SamplerConfig(temperature=0)) for n in (3, 1, 5, 2, 4)]
    prompts = [[1] * 5, [2] * 9, [3], [4] * 2, [5] * 7]
    seen = []
    results, stats = generate(eng, samp, prompts, cfgs, on_token=lambda i, t: seen.append((i, t)))
    assert [len(r.tokens) for r in results] == [3, 1, 5, 2, 4]
    assert all(r.finish_reason == "length" for r in results)
    assert results[0].tokens == [105, 106, 107] and results[2].tokens == [101, 102, 103, 104, 105]
    assert stats.batches == 2 and stats.output_tokens == 15 and len(seen) == 15        # one call per token
    assert [t for i, t in seen if i == 4] == results[4].tokens
    # first batch: three prompts in one step with the last place wanted, then one token each for the living
    assert eng.steps[0] == [(0, [1] * 5, [4]), (1, [2] * 9, [8]), (2, [3], [0])]
    assert eng.steps[1] == [(0, [105], [0]), (2, [101], [0])]                          # request 1 ended after one token
    assert eng.steps[3] == [(2, [103], [0])]
    # no step feeds a sequence's last token back; the second batch runs in slots the first gave back
    assert sum(len(s) for s in eng.steps) == 3 + 2 + 2 + 1 + 1 + 2 + 2 + 1 + 1
    assert sorted(eng.closed) == [0, 0, 1, 1, 2] and not eng.held and eng.free_slots() == 3
    # a time for every step: a prompt step and then one per choice, for each batch
    assert stats.steps == len(eng.steps) and len(stats.step_ms) == 2 + samp.waited and all(t >= 0 for t in stats.step_ms)


def test_loop_runs_a_step_ahead_and_drops_the_step_of_a_sequence_that_stopped():
    """The step that feeds a token is queued before the token is known.  A stop token is therefore fed once, in the step
    that was already on its way; that step's row is dropped, nothing of it is emitted, the slot goes back, and the rows
    of the sequences that go on are picked out of the result by their place among the sequences that were fed."""
    eng = FakeEngine()
    samp = ScriptSampler(stop_at={(0, 7): 2, (1, 3): 9})      # request 0 stops at its third choice, request 1 at once
    cfg = GenerateConfig(max_tokens=6, sampler=SamplerConfig(temperature=0))
    results, stats = generate(eng, samp, [[1] * 5, [1] * 3, [1] * 2], [cfg] * 3, default_stop=(2, 9))
    assert results[0].tokens == [105, 106] and results[0].finish_reason == "stop"
    assert results[1].tokens == [] and results[1].finish_reason == "stop"             # immediate stop: nothing
    assert results[2].tokens == [102, 103, 104, 105, 106, 107] and results[2].finish_reason == "length"
    # step 1 was queued for all three before request 1's stop was known; request 1 is not in step 2
    assert [slot for slot, _, _ in eng.steps[1]] == [0, 1, 2] and eng.steps[1][1][1] == [9]
    assert [slot for slot, _, _ in eng.steps[2]] == [0, 2]
    # request 0's stop token (2) went into step 3, the step after it only has request 2
    assert eng.steps[3] == [(0, [2], [0]), (2, [104], [0])] and [slot for slot, _, _ in eng.steps[4]] == [2]
    # the sampler never saw a row of a sequence that had stopped, and rows stayed with their sequences
    for rows, _, _ in samp.calls[1:]:
        assert all((slot, n) != (1, 4) for slot, n in rows)
    assert samp.calls[3][0] == [(2, 5)]
    assert stats.output_tokens == 8 and not eng.held and sorted(eng.closed) == [0, 1, 2]
    # the same script with ignore_eos runs to the length
    cfg2 = GenerateConfig(max_tokens=6, sampler=SamplerConfig(temperature=0), ignore_eos=True)
    r2, _ = generate(FakeEngine(), ScriptSampler(stop_at={(0, 7): 2}), [[1] * 5], [cfg2], default_stop=(2,))
    assert len(r2[0].tokens) == 6 and 2 in r2[0].tokens
    # a request's own stop set replaces the model's
    cfg3 = GenerateConfig(max_tokens=6, sampler=SamplerConfig(temperature=0), stop_tokens=(106,))
    r3, _ = generate(FakeEngine(), ScriptSampler(), [[1] * 5], [cfg3], default_stop=(105,))
    assert r3[0].tokens == [105] and r3[0].finish_reason == "stop"


def test_loop_context_end_and_errors():
    eng = FakeEngine(max_ctx=16, pages=4)
    cfg = GenerateConfig(max_tokens=100, sampler=SamplerConfig(temperature=0))
    results, _ = generate(eng, ScriptSampler(), [[1] * 10], [cfg])
    assert results[0].finish_reason == "context" and len(results[0].tokens) == 5      # stops when 15 tokens are cached
    assert eng.steps[-1] == [(0, [113], [0])] and len(eng.steps) == 5                  # the fifth token is not fed: nothing follows it
    with pytest.raises(GenerationError, match="prompt too long: 16 tokens"):
        generate(eng, ScriptSampler(), [[1] * 16], [cfg])
    with pytest.raises(GenerationError, match="empty prompt"):
        generate(eng, ScriptSampler(), [[]], [cfg])
    with pytest.raises(GenerationError, match="do not fit"):
        generate(FakeEngine(max_ctx=4096, pages=1), ScriptSampler(), [[1] * 70], [cfg])
    zero, _ = generate(eng, ScriptSampler(), [[1] * 3], [GenerateConfig(max_tokens=0)])
    assert zero[0].tokens == [] and zero[0].finish_reason == "length" and not eng.held
    # a prompt that fills the context but for one place: nothing can be chosen
    full, _ = generate(eng, ScriptSampler(), [[1] * 15], [cfg])
    assert full[0].tokens == [] and full[0].finish_reason == "context" and not eng.held


def test_loop_gives_slots_back_when_a_step_fails():
    class Failing(FakeEngine):
        def decode(self, slots, ids):
            if len(self.steps) == 2:
                raise RuntimeError("boom")
            return super().decode(slots, ids)
    eng = Failing()
    cfg = GenerateConfig(max_tokens=5, sampler=SamplerConfig(temperature=0))
    with pytest.raises(RuntimeError, match="boom"):
        generate(eng, ScriptSampler(), [[1] * 5, [1] * 2], [cfg, cfg])
    assert not eng.held and eng.free_slots() == 3


def test_draws_are_per_request_and_seeded():
    samp = ScriptSampler()
    cfg = GenerateConfig(max_tokens=3, seed=77)
    generate(FakeEngine(), samp, [[1] * 4, [1] * 2], [cfg, cfg])
    u0 = [c[1] for c in samp.calls]
    assert u0[0] == [uniform(77, 0, 0), uniform(77, 1, 0)] and u0[2] == [uniform(77, 0, 2), uniform(77, 1, 2)]
    assert all(0.0 <= x < 1.0 for call in u0 for x in call)
    assert np.float32(u0[1][0]) == u0[1][0]                      # representable in float32
    assert samp.calls[2][2] == [[104, 105], [102, 103]]          # the tokens so far, kept under each request's key
    vals = [uniform(1, 0, s) for s in range(4000)]
    assert abs(np.mean(vals) - 0.5) < 0.02 and len(set(vals)) > 3990


def test_options_have_the_reference_defaults_and_meanings():
    """ops/sampling.go:19-27, models/llm/generate.go:25-31, dlgo.go:213-248."""
    d = apply_options([])
    assert (d.max_tokens, d.seed) == (256, -1)
    s = d.sampler
    assert (s.temperature, s.top_k, s.top_p, s.min_p, s.repetition_penalty) == (0.7, 40, 0.9, 0.0, 1.1)
    c = apply_options([with_max_tokens(5), with_temperature(0.3), with_top_k(7), with_top_p(0.5), with_seed(9)])
    assert (c.max_tokens, c.sampler.temperature, c.sampler.top_k, c.sampler.top_p, c.seed) == (5, 0.3, 7, 0.5, 9)
    assert apply_options([with_greedy()]).sampler.greedy and apply_options([with_temperature(0)]).sampler.greedy
    assert apply_options([]).sampler is not apply_options([]).sampler
    with pytest.raises(ValueError):
        apply_options([with_temperature(-1)])
    import dlgo_amd
    assert dlgo_amd.WithMaxTokens is dlgo_amd.with_max_tokens and dlgo_amd.LoadLLM is dlgo_amd.load_llm


def test_prompts_are_integer_token_ids():
    """The entry point takes ids of any integer kind and tells one prompt from a list of prompts by its first element;
    floats and text are refused rather than cut down to integers."""
    from dlgo_amd.api import _ids, _is_id
    assert _ids([1, np.int64(2), torch.tensor(3)], 0) == [1, 2, 3] and _ids(np.array([4, 5]), 0) == [4, 5]
    assert _is_id(7) and _is_id(np.int32(7)) and _is_id(torch.tensor([7, 8])[0])
    assert not _is_id([7]) and not _is_id(7.0) and not _is_id("7")
    for bad in ([1.5, 2.0], "hello", [[1, 2]], [None]):
        with pytest.raises(GenerationError, match="request 3: a prompt is a sequence of integer token ids"):
            _ids(bad, 3)


def test_command_line_checks_like_the_reference(capsys):
    """examples/simple_chat/main.go:28-39."""
    from dlgo_amd.cli import main
    assert main(["--ctx", "0", "x"]) == 1 and "--ctx must be > 0" in capsys.readouterr().err
    assert main(["--max-tokens", "0", "x"]) == 1 and "--max-tokens must be > 0" in capsys.readouterr().err
    assert main(["--temp", "-0.1", "x"]) == 1 and "--temp must be >= 0" in capsys.readouterr().err
    assert main(["x", "--prompt-ids", "1,b,3"]) == 1 and "Error reading prompts" in capsys.readouterr().err
    assert main(["x", "--prompts-file", "/nonexistent/prompts.txt"]) == 1 and "Error reading prompts" in capsys.readouterr().err


def test_command_line_writes_a_random_model_or_says_why_not(tmp_path, capsys):
    import json
    from conftest import TINY_A
    from dlgo_amd.cli import main
    from dlgo_amd.config import load_config
    raw = {k: v for k, v in TINY_A.items() if k != "initializer_range"}
    (tmp_path / "c.json").write_text(json.dumps(raw))
    out = str(tmp_path / "m")
    assert main(["--write-random", str(tmp_path / "c.json"), out]) == 1
    assert "initializer_range" in capsys.readouterr().err          # no width of the weights in the file: one line, no traceback
    assert main(["--write-random", str(tmp_path / "c.json"), out, "--weight-std", "0.05", "--weight-seed", "3"]) == 0
    assert load_config(out).hidden_size == raw["hidden_size"] and (tmp_path / "m" / "model.safetensors").exists()
    assert main(["--write-random", str(tmp_path / "nope.json"), out]) == 1 and "no such file" in capsys.readouterr().err


def test_command_line_takes_a_folder_or_a_configuration_to_draw_weights_for(tmp_path, capsys):
    """Exactly one of MODEL_DIR and --random-config; without a GPU either ends in one line that says so, no traceback."""
    import json
    from conftest import TINY_A
    from dlgo_amd.cli import main
    (tmp_path / "c.json").write_text(json.dumps(TINY_A))
    for argv in ([], ["x", "--random-config", str(tmp_path / "c.json")]):
        with pytest.raises(SystemExit) as e:
            main(argv)
        assert e.value.code == 2 and "one of them" in capsys.readouterr().err
    if not torch.cuda.is_available():
        assert main(["--random-config", str(tmp_path / "c.json"), "--weight-seed", "3", "--prompt-ids", "1,2"]) == 1
        err = capsys.readouterr().err
        assert err.startswith("Error loading model:") and "no HIP device" in err and "Traceback" not in err
    assert main(["--random-config", str(tmp_path / "missing.json")]) == 1 and "Error loading model" in capsys.readouterr().err


def test_replay_program_checks_its_arguments_before_anything_else(tmp_path):
    """bin/trace_run takes exactly one of --model and --config and a positive --max-tokens; a model that cannot be
    loaded (here: no GPU) ends in one line and status 1, an empty input in status 0 only after a model is there."""
    import json
    import subprocess
    import sys
    from pathlib import Path
    from conftest import TINY_A
    prog = str(Path(__file__).resolve().parents[1] / "bin" / "trace_run")
    (tmp_path / "c.json").write_text(json.dumps(TINY_A))
    common = ["--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "64"]

    def run(*argv):
        return subprocess.run([sys.executable, prog, *argv], input="", capture_output=True, text=True, timeout=300)
    r = run(*common)
    assert r.returncode == 2 and "one of --model DIR and --config FILE" in r.stderr
    r = run("--model", str(tmp_path), "--config", str(tmp_path / "c.json"), *common)
    assert r.returncode == 2 and "one of --model DIR and --config FILE" in r.stderr
    r = run("--config", str(tmp_path / "c.json"), "--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "0")
    assert r.returncode == 2 and "--max-tokens must be > 0" in r.stderr
    if not torch.cuda.is_available():
        r = run("--config", str(tmp_path / "c.json"), "--weight-seed", "3", *common)
        assert r.returncode == 1 and "trace_run: cannot load" in r.stderr and "no HIP device" in r.stderr
        assert "Traceback" not in r.stderr


def test_engine_refuses_to_run_without_a_gpu(tmp_path):
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from conftest import TINY_A, make_folder
    from dlgo_amd.engine import Engine, EngineError
    folder = make_folder(TINY_A, 1, tmp_path)
    with pytest.raises(EngineError, match="no HIP device"):
        Engine.from_folder(folder, "float32")
