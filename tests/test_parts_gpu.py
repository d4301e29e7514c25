"""Each part alone against the plain implementation, and the generality of the assembly: a toy
mixer with state of its own, a toy feed-forward that routes each row to one of several experts, a toy
position encoding, a windowed attention layer and a run order that names a layer twice and lets a
run read another run's cache, all registered from here,
built by the registry and stepped by the engine without a change to the library's files."""
import math
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional

import numpy as np
import pytest
import torch

import plain_llama as plain
from conftest import TINY_B

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _Ctx:
    """The least a part needs of a step: buffers, the cache and the step's arrays."""

    def __init__(self, dtype, unit_needs, seq_lens, starts, max_tokens=1024, max_ctx=512):
        from dlgo_amd.cache import Cache
        from dlgo_amd.engine.context import Workspace
        self.dtype, self.device = dtype, torch.device(DEV)
        self.cache = Cache(unit_needs, max_tokens, max_ctx, dtype, DEV)
        self.workspace = Workspace(self.device, 1024)
        self.engine = self
        self.rows(seq_lens, starts, first=True)

    def rows(self, q_lens, starts, first=False, slots=None):
        if first:
            self.all_slots = [self.cache.alloc_slot() for _ in q_lens][::-1]
        self.step_slots = list(slots) if slots is not None else list(self.all_slots)
        self.cache.reserve([(s, st + q) for s, st, q in zip(self.step_slots, starts, q_lens)])
        self.cache.sync_tables()
        i32 = lambda v: torch.tensor(list(v), dtype=torch.int32, device=DEV)
        self.positions = i32(p for st, q in zip(starts, q_lens) for p in range(st, st + q))
        self.tok_seq = i32(i for i, q in enumerate(q_lens) for _ in range(q))
        self.slots, self.start_pos = i32(self.step_slots), i32(starts)
        self.cu_q = i32(np.concatenate([[0], np.cumsum(q_lens)]))
        self.host = {"q_lens": np.array(q_lens), "start_pos": np.array(starts), "slots": np.array(self.step_slots)}
        self.n_seq, self.n_tokens, self.max_pages_used = len(q_lens), int(sum(q_lens)), None
        self.max_q_len = max(q_lens)

    def done(self):
        for s, q in zip(self.step_slots, self.host["q_lens"]):
            self.cache.advance(int(s), int(q))

    def buffer(self, name, shape, dtype):
        return self.workspace.get(name, shape, dtype)

    def scratch(self, name, n, dtype, zero=False):
        return self.workspace.flat(name, n, dtype, zero)


def _rel(got, want):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    return np.abs(got - want).max() / (np.abs(want).max() + 1e-30)


TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_embedding_head_feed_forward_alone(dtype):
    from dlgo_amd.parts import Embedding, GatedFeedForward, OutputHead, RMSNorm
    g = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g)
    ctx = _Ctx(dtype, [], [7], [0])
    # norm
    norm = RMSNorm(40, 1e-3)
    norm.load({"weight": 1 + 0.2 * r(40)}, DEV, dtype)
    x = (3 * r(7, 40)).to(DEV)
    out = torch.empty(7, 40, dtype=dtype, device=DEV)
    norm(x, out)
    assert _rel(out, plain.rmsnorm(x.double().cpu().numpy(), norm.weight.double().cpu().numpy(), 1e-3)) <= TOL[dtype]
    # embedding and a head tied to it
    emb = Embedding(50, 40)
    emb.load({"weight": r(50, 40).to(dtype)}, DEV, dtype)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    rows = torch.empty(4, 40, device=DEV)
    emb(ids, rows)
    assert torch.equal(rows.cpu(), emb.weight.float().cpu()[ids.cpu().long()])
    head = OutputHead(50, 40, tied_to=emb)
    assert head.tensor_specs() == {} and head.weight is emb.weight
    xn = r(4, 40).to(dtype).to(DEV)
    logits = torch.empty(4, 50, device=DEV)
    head(xn, logits)
    assert _rel(logits, xn.double().cpu().numpy() @ emb.weight.double().cpu().numpy().T) <= 1e-5
    # gated feed-forward, adding into the residual
    ffn = GatedFeedForward(40, 88, "silu")
    w = {"gate_proj.weight": r(88, 40).to(dtype), "up_proj.weight": r(88, 40).to(dtype), "down_proj.weight": (0.2 * r(40, 88)).to(dtype)}
    ffn.load(w, DEV, dtype)
    res = r(4, 40).to(DEV)
    res0 = res.double().cpu().numpy()
    ffn.forward(xn, ctx, res)
    want = res0 + plain.feed_forward(xn.double().cpu().numpy(), *(w[k].double().numpy() for k in
                                                                  ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    assert _rel(res, want) <= TOL[dtype]


def test_rotary_tables_follow_the_configuration():
    from dlgo_amd.config import config_from_dict
    from dlgo_amd.parts import Rotary
    cfg = config_from_dict(TINY_B)
    rot = Rotary(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling)
    rot.prepare(300, torch.device(DEV))
    inv = plain.rope_inv_freq(32, 500000.0, TINY_B["rope_scaling"])
    assert np.array_equal(rot.frequencies, inv)
    table = rot.rotation()
    ang = np.arange(300)[:, None] * inv[None]
    # float64 angles, rounded once (the tables are shared by everyone with this recipe, so they may be longer than asked)
    assert np.array_equal(table.cos.cpu().numpy()[:300], np.cos(ang).astype(np.float32))
    assert np.array_equal(table.sin.cpu().numpy()[:300], np.sin(ang).astype(np.float32))
    assert table.cos.shape[0] >= 300 and table.cos.shape[1] == 16 and not table.interleaved and table.width == 32
    plain_rot = Rotary(32, 500000.0, None)
    assert not np.array_equal(plain_rot.frequencies, inv)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 37])
@pytest.mark.parametrize("between", [False, True])
def test_attention_part_alone(dtype, window, between):
    """Whole rows, then a continuation in pieces, for two sequences of unequal lengths, against plain attention with rotation.
    between: the layer also has what the reference puts between projection and rotation where a layer's tensors ask
    for it (models/llm/forward.go:227-244): biases of the projections, and an RMSNorm of every q and k head over the
    head's own elements; the output projection has a bias too."""
    from dlgo_amd.parts import Attention, Rotary
    H, KV, hd, d = 6, 2, 32, 48
    eps = 1e-4
    g = torch.Generator().manual_seed(1)
    r = lambda *s: torch.randn(*s, generator=g)
    extra = dict(bias=True, out_bias=True, qk_norm_eps=eps) if between else {}
    att = Attention(d, H, KV, hd, Rotary(hd, 10000.0), window=window, **extra)
    w = {"q_proj.weight": (0.3 * r(H * hd, d)).to(dtype), "k_proj.weight": (0.3 * r(KV * hd, d)).to(dtype),
         "v_proj.weight": (0.3 * r(KV * hd, d)).to(dtype), "o_proj.weight": (0.2 * r(d, H * hd)).to(dtype)}
    if between:
        w.update({"q_proj.bias": r(H * hd).to(dtype), "k_proj.bias": r(KV * hd).to(dtype), "v_proj.bias": (0.5 * r(KV * hd)).to(dtype),
                  "o_proj.bias": (0.5 * r(d)).to(dtype), "q_norm.weight": (1 + 0.3 * r(hd)).to(dtype), "k_norm.weight": (1 + 0.3 * r(hd)).to(dtype)})
    assert set(att.tensor_specs()) == set(w)
    att.load(w, DEV, dtype)
    att.prepare(512, torch.device(DEV))
    lens = [100, 70]
    xs = [r(n, d).to(dtype) for n in lens]
    inv = plain.rope_inv_freq(hd, 10000.0)
    f64 = lambda name: w[name].double().numpy()
    want = []
    for x in xs:
        xd = x.double().numpy()
        q, k, v = (xd @ f64(n).T for n in ("q_proj.weight", "k_proj.weight", "v_proj.weight"))
        if between:
            q, k, v = q + f64("q_proj.bias"), k + f64("k_proj.bias"), v + f64("v_proj.bias")
            q = plain.rmsnorm(q.reshape(-1, H, hd), f64("q_norm.weight"), eps).reshape(-1, H * hd)
            k = plain.rmsnorm(k.reshape(-1, KV, hd), f64("k_norm.weight"), eps).reshape(-1, KV * hd)
        for t in range(len(xd)):
            q[t] = plain.rope_apply(q[t].reshape(H, hd), t, inv).reshape(-1)
            k[t] = plain.rope_apply(k[t].reshape(KV, hd), t, inv).reshape(-1)
        out = plain.attention(q, k, v, H, KV, hd, window) @ f64("o_proj.weight").T
        want.append(out + f64("o_proj.bias") if between else out)
    ctx = _Ctx(dtype, [att.cache_needs()], [60, 70], [0, 0])
    # (sequences in the step, their rows, their starts): both whole-ish, then the first goes on alone: a piece, a single row
    steps = [([0, 1], [60, 70], [0, 0]), ([0], [39], [60]), ([0], [1], [99])]
    got = [[], []]
    for n, (who, q_lens, starts) in enumerate(steps):
        if n:
            ctx.rows(q_lens, starts, slots=[ctx.all_slots[i] for i in who])
        x = torch.cat([xs[i][st:st + q] for i, q, st in zip(who, q_lens, starts)]).to(DEV)
        res = torch.zeros(x.shape[0], d, device=DEV)
        att.forward(x, ctx, 0, res)
        ctx.done()
        o = 0
        for i, q in zip(who, q_lens):
            got[i].append(res[o:o + q].double().cpu().numpy())
            o += q
    for i in range(2):
        assert _rel(np.concatenate(got[i]), want[i]) <= TOL[dtype] * 2, (i, window)


# ---------------------------------------------------------------------------
# a toy architecture, defined here, built by the registry, stepped by the engine
# ---------------------------------------------------------------------------
def _register_toy():
    from dlgo_amd.config import KeyReader, ModelConfig, register_architecture
    from dlgo_amd.parts import (CacheNeed, DecoderModel, Embedding, FeedForward, LayerRun, Mixer, OutputHead,
                                PositionEncoding, TensorSpec, make_part, register_part, stored)

    class DecayMixer(Mixer):
        """A mixer with state of its own: s_t = decay * s_{t-1} + x_t per sequence, out_t = W s_t.
        The state lives in the cache's per-slot state area; rows of a sequence are taken in order."""

        graph_safe = False       # forward() walks the step's host-side lengths and slots: nothing to record and replay

        def __init__(self, width, decay):
            self.width, self.decay = width, decay

        def tensor_specs(self):
            return {"mix.weight": TensorSpec((self.width, self.width))}

        def cache_needs(self):
            return [CacheNeed(kind="state", state_shape=(self.width,), state_dtype=torch.float32)]

        def load(self, tensors, device, dtype):
            self.w = stored(tensors["mix.weight"], self.tensor_specs()["mix.weight"], device, torch.float32)

        def forward(self, xn, ctx, unit, residual, owns_cache=True):
            state = ctx.cache.state_of(unit)
            x = xn.float()
            q_lens, slots = ctx.host["q_lens"], ctx.host["slots"]
            o = 0
            for n, slot in zip(q_lens, slots):
                s = state[int(slot)].clone()
                for t in range(o, o + int(n)):
                    s = self.decay * s + x[t]
                    residual[t] += s @ self.w.T
                state[int(slot)] = s
                o += int(n)

    class RoutedFeedForward(FeedForward):
        """A feed-forward with routing: a float32 router scores the experts, each row goes to its best one.  The
        experts are the library's gated feed-forwards, mounted under experts.<e>; every expert runs on every row and
        the rows it was not chosen for are masked, which is slow and has no step that depends on the data."""

        def __init__(self, width, inner, n_experts):
            self.width, self.n_experts = width, n_experts
            self.experts = [make_part("feed_forward", "gated", width, inner, "silu") for _ in range(n_experts)]

        def tensor_specs(self):
            specs = {"router.weight": TensorSpec((self.n_experts, self.width), kind="vector")}
            for e, expert in enumerate(self.experts):
                specs.update({f"experts.{e}.{n}": sp for n, sp in expert.tensor_specs().items()})
            return specs

        def kernel_variants(self, dtype):
            return [v for expert in self.experts for v in expert.kernel_variants(dtype)]

        def check(self, dtype):
            for expert in self.experts:
                expert.check(dtype)

        def load(self, tensors, device, dtype):
            self.router = stored(tensors["router.weight"], self.tensor_specs()["router.weight"], device, dtype)
            for e, expert in enumerate(self.experts):
                pre = f"experts.{e}."
                expert.load({n[len(pre):]: t for n, t in tensors.items() if n.startswith(pre)}, device, dtype)

        def forward(self, xn, ctx, residual, norm=None):
            choice = (xn.float() @ self.router.T).argmax(-1)          # router logits in float32
            for e, expert in enumerate(self.experts):
                mine = ctx.buffer("toy.expert_out", tuple(residual.shape), torch.float32)
                mine.zero_()
                expert.forward(xn, ctx, mine)
                residual += mine * (choice == e).unsqueeze(1)

    class LearnedPosition(PositionEncoding):
        """Another position encoding: a learned vector per position, added to the embedded rows."""

        def __init__(self, max_positions, width):
            self.max_positions, self.width = max_positions, width

        def tensor_specs(self):
            return {"weight": TensorSpec((self.max_positions, self.width))}

        def load(self, tensors, device, dtype):
            self.table = stored(tensors["weight"], TensorSpec((self.max_positions, self.width), kind="vector"), device, dtype)

        def on_embedding(self, x, ctx):
            x += self.table[ctx.positions.long()]

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int
        width: int
        heads: int
        kv_heads: int
        head_dim: int
        inner: int
        experts: int
        eps: float
        decay: float
        window: int
        table_rows: int              # rows of the learned position table: what bounds a sequence here
        spread: float

        # what the library asks of a configuration; it reads none of the keys above itself
        def context_length(self):
            return self.table_rows

        def storage_dtype(self):
            return "float32"

        def init_std(self):
            return self.spread

        @classmethod
        def from_dict(cls, raw: Mapping[str, Any]):
            r = KeyReader(raw)
            vals = dict(architecture=raw["architectures"][0], vocab_size=r.integer("vocab_size"), width=r.integer("width"),
                        heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), head_dim=r.integer("head_dim"),
                        inner=r.integer("inner"), experts=r.integer("experts"), eps=r.number("eps"), decay=r.number("decay"), window=r.integer("window"),
                        table_rows=r.integer("table_rows"), spread=r.number("spread"))
            r.finish()
            return cls(**vals)

        def to_dict(self) -> Dict[str, Any]:
            d = dict(self.__dict__)
            d["architectures"] = [d.pop("architecture")]
            return d

    def build(cfg: ToyConfig):
        d = cfg.width
        norm = lambda: make_part("norm", "rmsnorm", d, cfg.eps)
        ffn = lambda: make_part("feed_forward", "gated", d, cfg.inner, "silu")

        def attention(window):
            return make_part("mixer", "attention", d, cfg.heads, cfg.kv_heads, cfg.head_dim, make_part("position", "none"),
                             window=window)
        mixers = [attention(None), make_part("mixer", "toy_decay", d, cfg.decay), attention(cfg.window)]
        # the layer with the state mixer routes its feed-forward; the attention layers have the dense one
        ffns = [ffn(), make_part("feed_forward", "toy_routed", d, cfg.inner, cfg.experts), ffn()]
        layers = [(f"blocks.{i}", make_part("block", "pre_norm", ("n1", norm()), ("mixer", m), ("n2", norm()), ("ff", f)))
                  for i, (m, f) in enumerate(zip(mixers, ffns))]
        emb = Embedding(cfg.vocab_size, d)
        # layer 1 (state) runs twice, each run with state of its own; the last run is layer 0 again, reading the
        # keys and values that the first run stored
        order = [LayerRun(0), LayerRun(1), LayerRun(2), LayerRun(1), LayerRun(0, reads_cache_of=0)]
        return DecoderModel(cfg, ("embed", emb), layers, ("final_norm", norm()), ("head", OutputHead(cfg.vocab_size, d, emb)),
                            order=order,
                            position=("positions", make_part("position", "toy_learned", cfg.table_rows, d)))

    register_part("mixer", "toy_decay", DecayMixer)
    register_part("feed_forward", "toy_routed", RoutedFeedForward)
    register_part("position", "toy_learned", LearnedPosition)
    register_architecture("ToyForCausalLM", ToyConfig, build)


TOY = {"architectures": ["ToyForCausalLM"], "vocab_size": 90, "width": 48, "heads": 3, "kv_heads": 1, "head_dim": 16, "inner": 72,
       "experts": 3, "eps": 1e-4, "decay": 0.8, "window": 20, "table_rows": 256, "spread": 0.15}


_EXPERTS_SEEN = set()        # the experts that the plain router chose, over all sequences of the test


def _toy_plain(w, tokens):
    """The toy model in plain float64 NumPy, whole sequence, no cache."""
    c = TOY
    d, H, KV, hd = c["width"], c["heads"], c["kv_heads"], c["head_dim"]
    x = w["embed.weight"][tokens] + w["positions.weight"][:len(tokens)]

    def att(x, i, window, kv_from=None):
        p = f"blocks.{i}."
        xn = plain.rmsnorm(x, w[p + "n1.weight"], c["eps"])
        q = xn @ w[p + "mixer.q_proj.weight"].T
        src = xn if kv_from is None else kv_from
        k, v = src @ w[p + "mixer.k_proj.weight"].T, src @ w[p + "mixer.v_proj.weight"].T
        h = x + plain.attention(q, k, v, H, KV, hd, window) @ w[p + "mixer.o_proj.weight"].T
        return ffn(h, p), xn

    def ffn(h, p):
        hn = plain.rmsnorm(h, w[p + "n2.weight"], c["eps"])
        if p + "ff.router.weight" not in w:
            return h + plain.feed_forward(hn, w[p + "ff.gate_proj.weight"], w[p + "ff.up_proj.weight"], w[p + "ff.down_proj.weight"])
        choice = (hn @ w[p + "ff.router.weight"].T).argmax(-1)
        _EXPERTS_SEEN.update(choice.tolist())
        out = h.copy()
        for t, e in enumerate(choice):
            q = f"{p}ff.experts.{e}."
            out[t] += plain.feed_forward(hn[t:t + 1], w[q + "gate_proj.weight"], w[q + "up_proj.weight"], w[q + "down_proj.weight"])[0]
        return out

    def decay(x):
        p = "blocks.1."
        xn = plain.rmsnorm(x, w[p + "n1.weight"], c["eps"])
        s, h = np.zeros(d), x.copy()
        for t in range(len(x)):
            s = c["decay"] * s + xn[t]
            h[t] += w[p + "mixer.mix.weight"] @ s
        return ffn(h, p)
    x, first_in = att(x, 0, None)
    x = decay(x)
    x, _ = att(x, 2, c["window"])
    x = decay(x)
    x, _ = att(x, 0, None, kv_from=first_in)      # queries from here, keys and values as the first run stored them
    return plain.rmsnorm(x, w["final_norm.weight"], c["eps"]) @ w["embed.weight"].T


def test_toy_architecture_is_registered_built_and_stepped(tmp_path):
    _register_toy()
    from dlgo_amd.config import config_from_dict
    from dlgo_amd.engine import Engine, Entry
    from dlgo_amd.weights import write_random_model
    cfg = config_from_dict(TOY)
    folder = write_random_model(cfg, 3, str(tmp_path), norm_jitter=0.1)
    _, w = plain.read_model(folder)
    # recording is asked for (the default), but one part says its launches depend on host-side numbers: every step runs as it is
    eng = Engine.from_folder(folder, "float32", max_tokens=1024, use_graphs=True)
    assert not eng.use_graphs and eng.eager_because == ["blocks.1.mixer"]
    assert len(eng.cache.groups) == 2 and len(eng.cache.state) == 2           # full and windowed keys/values; two runs with state
    assert eng.model.run_unit == [0, 1, 2, 3, 0] and eng.model.run_owns == [True, True, True, True, False]
    rng = np.random.default_rng(0)
    seqs = [rng.integers(0, 90, size=n).tolist() for n in (90, 30, 1)]
    want = [_toy_plain(w, s) for s in seqs]
    assert _EXPERTS_SEEN == set(range(TOY["experts"]))             # the routing is exercised: every expert gets rows
    # whole, in one batch of unequal lengths
    slots = eng.open(3)
    out = eng.step([Entry(s, t, list(range(len(t)))) for s, t in zip(slots, seqs)]).cpu().numpy()
    o = 0
    for t, wnt in zip(seqs, want):
        assert _rel(out[o:o + len(t)], wnt) <= 2e-5
        o += len(t)
    eng.close(slots)
    # a prompt, then one token at a time: the state and both caches carry over; the slot was used before
    (slot,) = eng.open(1)
    got = [eng.step([Entry(slot, seqs[0][:50], list(range(50)))]).cpu().numpy()]
    for t in seqs[0][50:]:
        got.append(eng.step([Entry(slot, [t], [0])]).cpu().numpy())
    assert _rel(np.concatenate(got), want[0]) <= 2e-5
    assert not eng._graphs
    eng.close([slot])
    eng.cache.check_consistent()
