"""The engine against the plain implementation: each request alone and whole; with its last
tokens one by one; in batches of unequal lengths whose shorter requests end earlier, one batch
after another so that slots are used again; in float32 and in bfloat16."""
import numpy as np
import pytest
import torch

import plain_llama as plain
from conftest import TINY_A, TINY_B, TINY_C, TINY_D, make_folder

pytestmark = pytest.mark.gpu

CONFIGS = {"A": (TINY_A, dict()), "B": (TINY_B, dict(norm_jitter=0.1)), "C": (TINY_C, dict(norm_jitter=0.1, std=0.12)),
           "D": (TINY_D, dict(norm_jitter=0.2, std=0.08))}
# float32: the engine against float64 arithmetic on the same weights; bfloat16: against the same,
# with the rounding of activations to 8 bits of mantissa at every layer
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (raw, kw) in CONFIGS.items():
        for wdtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"tiny{name}_{wdtype}")
            make_folder(raw, seed=11 + len(out), path=d, dtype=wdtype, **kw)
            out[name, wdtype] = str(d)
    return out


@pytest.fixture(scope="module")
def oracle(folders):
    cache = {}

    def get(name, wdtype, tokens):
        key = (name, wdtype, tuple(tokens))
        if key not in cache:
            cfg, w = plain.read_model(folders[name, wdtype])
            cache[key] = plain.forward(cfg, w, tokens)
        return cache[key]
    return get


def engine_for(folder, dtype, **kw):
    from dlgo_amd.engine import Engine
    kw.setdefault("max_tokens", 2048)
    return Engine.from_folder(folder, dtype, **kw)


def rel_err(got, want):
    got = np.asarray(got, dtype=np.float64)
    return np.abs(got - want).max() / (np.abs(want).max() + 1e-30)


def prompts_for(raw, lens, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, raw["vocab_size"], size=n).tolist() for n in lens]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_prompt(folders, oracle, name, dtype):
    from dlgo_amd.engine import Entry
    raw = CONFIGS[name][0]
    wdtype = dtype
    eng = engine_for(folders[name, wdtype], dtype)
    for tokens in prompts_for(raw, [1, 5, 70, 127], seed=3):
        (slot,) = eng.open(1)
        logits = eng.step([Entry(slot, tokens, list(range(len(tokens))))]).cpu().numpy()
        eng.close([slot])
        want = oracle(name, wdtype, tokens)
        assert logits.shape == want.shape
        assert np.isfinite(logits).all()
        assert rel_err(logits, want) <= TOL[dtype], (name, dtype, len(tokens))
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("graphs", [False, True])
def test_last_tokens_one_by_one(folders, oracle, name, dtype, graphs):
    from dlgo_amd.engine import Entry
    raw = CONFIGS[name][0]
    eng = engine_for(folders[name, dtype], dtype, use_graphs=graphs)
    (tokens,) = prompts_for(raw, [100], seed=5)
    want = oracle(name, dtype, tokens)
    (slot,) = eng.open(1)
    head = len(tokens) - 32
    # the results are looked at only after the last step: each step's logits are the caller's to keep
    rows = [eng.step([Entry(slot, tokens[:head], list(range(head)))])]
    for t in tokens[head:]:
        rows.append(eng.step([Entry(slot, [t], [0])]))
    got = np.concatenate([r.cpu().numpy() for r in rows])
    assert rel_err(got, want) <= TOL[dtype]
    # whole against one-by-one: the same numbers beyond rounding, also where the plain one is further away
    eng.close([slot])
    (slot,) = eng.open(1)
    whole = eng.step([Entry(slot, tokens, list(range(len(tokens))))]).cpu().numpy()
    assert rel_err(got, whole.astype(np.float64)) <= (1e-5 if dtype == "float32" else TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_unequal_batches_with_slot_reuse(folders, oracle, name, dtype):
    """Three batches one after another in a cache that holds one batch at a time; each batch's requests
    start together with unequal prompts, go on one token per step, and end at different times."""
    from dlgo_amd.engine import Entry
    raw = CONFIGS[name][0]
    eng = engine_for(folders[name, dtype], dtype, max_tokens=6 * 64, max_slots=4)
    batches = [[(5, 8), (9, 3), (1, 12)], [(17, 12), (3, 1), (40, 6), (1, 9)], [(64, 2), (63, 3), (65, 1)]]
    seed = 0
    for batch in batches:
        seed += 1
        seqs = prompts_for(raw, [p + d for p, d in batch], seed=seed)
        want = [oracle(name, dtype, s) for s in seqs]
        slots = eng.open(len(batch))
        got = [[] for _ in batch]
        out = eng.step([Entry(slots[i], seqs[i][:p], list(range(p))) for i, (p, d) in enumerate(batch)]).cpu().numpy()
        o = 0
        for i, (p, d) in enumerate(batch):
            got[i].append(out[o:o + p])
            o += p
        step = 0
        live = list(range(len(batch)))
        while live:
            live = [i for i in live if step < batch[i][1]]
            for i in range(len(batch)):
                if i not in live and slots[i] is not None and step >= batch[i][1]:
                    eng.close([slots[i]])
                    slots[i] = None
            if not live:
                break
            out = eng.step([Entry(slots[i], [seqs[i][batch[i][0] + step]], [0]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1].copy())
            step += 1
        eng.cache.check_consistent()
        assert eng.cache.n_free_slots == 4
        for i in range(len(batch)):
            g = np.concatenate(got[i])
            assert g.shape == want[i].shape
            assert rel_err(g, want[i]) <= TOL[dtype], (name, dtype, batch[i])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "D"])
def test_a_forked_sequence_goes_its_own_way(folders, oracle, name, dtype):
    """memory/kvcache.go:38-55 (Clone): a sequence is copied after its prompt (and one at an earlier length); the copies
    and the original then take different tokens in the same steps, and each gives the logits of its own whole
    sequence.  The original is closed half way: the copies hold nothing of it."""
    from dlgo_amd.engine import Entry
    raw = CONFIGS[name][0]
    eng = engine_for(folders[name, dtype], dtype, max_tokens=16 * 64, max_slots=4)
    prompt, = prompts_for(raw, [70], seed=11)
    tails = prompts_for(raw, [9, 9, 9], seed=12)
    (a,) = eng.open(1)
    eng.step([Entry(a, prompt, [])])
    b = eng.fork(a)
    c = eng.fork(a, 33)                       # not at a page's edge: the copy's last page holds tokens it must not see
    assert (eng.length(a), eng.length(b), eng.length(c)) == (70, 70, 33)
    seqs = {a: prompt + tails[0], b: prompt + tails[1], c: prompt[:33] + tails[2]}
    got = {s: [] for s in seqs}
    live = [a, b, c]
    for step in range(9):
        if step == 4:
            eng.close([a])
            live.remove(a)
        out = eng.step([Entry(s, [seqs[s][eng.length(s)]], [0]) for s in live]).cpu().numpy()
        for r, s in enumerate(live):
            got[s].append(out[r])
    eng.cache.check_consistent()
    for s, rows in got.items():
        want = oracle(name, dtype, seqs[s])
        first = len(seqs[s]) - 9
        assert rel_err(np.stack(rows), want[first:first + len(rows)]) <= TOL[dtype], (name, dtype, s)
    eng.close([b, c])
    assert eng.cache.n_free_slots == 4 and all(g.pool.n_free == g.pool.n_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_step_cut_into_pieces_and_batch_mates(folders, oracle, dtype):
    """A step with more rows than the workspace holds is cut along the rows; a request's logits do not
    depend on that nor on what else is in the batch."""
    from dlgo_amd.engine import Entry
    raw = TINY_B
    seqs = prompts_for(raw, [150, 33, 70], seed=9)
    big = engine_for(folders["B", dtype], dtype, max_step_tokens=4096)
    small = engine_for(folders["B", dtype], dtype, max_step_tokens=48)
    outs = []
    for eng in (big, small):
        slots = eng.open(3)
        outs.append(eng.step([Entry(s, t, list(range(len(t)))) for s, t in zip(slots, seqs)]).cpu().numpy())
    tol = 1e-5 if dtype == "float32" else TOL[dtype]
    assert rel_err(outs[1], outs[0].astype(np.float64)) <= tol
    o = 0
    for t in seqs:
        assert rel_err(outs[0][o:o + len(t)], oracle("B", dtype, t)) <= TOL[dtype]
        o += len(t)


LONG = dict(TINY_B, max_position_embeddings=8192, num_hidden_layers=2, num_key_value_heads=2,
            rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                          "original_max_position_embeddings": 1024})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_thousands_of_tokens(tmp_path, dtype):
    """Prompts of thousands of tokens, cut into pieces of 1024 rows, then 40 tokens one by one from recorded steps:
    dozens of pages a sequence, positions beyond the scaling's original length, pages dealt to several blocks.  The
    first sequence repeats one rare token far back and near the end, so that the late queries lean on a far key."""
    from dlgo_amd.engine import Entry
    folder = make_folder(LONG, seed=5, path=tmp_path, dtype=dtype, norm_jitter=0.1, std=0.08)
    cfg, w = plain.read_model(str(folder))
    rng = np.random.default_rng(4)
    lens, n_dec = [2500, 700, 65], 40
    seqs = [rng.integers(1, LONG["vocab_size"], size=n + n_dec).tolist() for n in lens]
    for at in (3, 2490, 2520):
        seqs[0][at] = 0
    want = [plain.forward(cfg, w, t) for t in seqs]
    eng = engine_for(str(folder), dtype, max_tokens=4096, max_ctx=4096, max_step_tokens=1024)
    slots = eng.open(3)
    got = [[eng.step([Entry(s, t[:n], [n - 2, n - 1]) for s, t, n in zip(slots, seqs, lens)]).cpu().numpy()]]
    for i in range(n_dec):
        got.append([eng.step([Entry(s, [t[n + i]], [0]) for s, t, n in zip(slots, seqs, lens)]).cpu().numpy()])
    tol = 5e-5 if dtype == "float32" else TOL[dtype]
    first = got[0][0]
    for j, (t, n) in enumerate(zip(seqs, lens)):
        assert rel_err(first[2 * j:2 * j + 2], want[j][n - 2:n]) <= tol, (dtype, "prompt", j)
        dec = np.stack([g[0][j] for g in got[1:]])
        assert rel_err(dec, want[j][n:n + n_dec]) <= tol, (dtype, "decode", j)
    eng.close(slots)
    eng.cache.check_consistent()


# -- tens of thousands of tokens ------------------------------------------------------------------------------------
# Two layers of Tiny B's widths with positions up to 32,768 and a scaling recipe whose original length is 1,024: at
# 20,000 tokens a sequence holds 313 pages, a decode step deals them to many blocks (more than a context of a few
# thousand tokens ever gives), and every rotary pair is far into the regime its wavelength puts it in.  Eight
# sequences of 100 to 20,000 tokens; the plain implementation follows each whole, once: the folder holds bfloat16
# weights, which a float32 run reads exactly, so both run dtypes have the same model before them.
FAR = dict(TINY_B, max_position_embeddings=32768, num_hidden_layers=2, num_key_value_heads=2,
           rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                         "original_max_position_embeddings": 1024})
FAR_LENS = [20000, 100, 300, 1000, 2100, 4200, 8300, 12000]
FAR_DECODE = 8


@pytest.fixture(scope="module")
def far(tmp_path_factory):
    folder = make_folder(FAR, seed=6, path=tmp_path_factory.mktemp("far"), dtype="bfloat16", norm_jitter=0.1, std=0.08)
    cfg, w = plain.read_model(str(folder))
    rng = np.random.default_rng(14)
    seqs = [rng.integers(1, FAR["vocab_size"], size=n + FAR_DECODE).tolist() for n in FAR_LENS]
    for at in (3, 9000, 19990, 20003):          # one rare token far back and near the end: late queries lean on far keys
        seqs[0][at] = 0
    # the prompt's last two rows and every decoded row
    want = [plain.forward(cfg, w, t, rows=range(n - 2, n + FAR_DECODE)) for t, n in zip(seqs, FAR_LENS)]
    return str(folder), seqs, want


def _prompt_then_tokens(eng, slots, seqs, lens, want, tol, what):
    from dlgo_amd.engine import Entry
    first = eng.step([Entry(s, t[:n], [n - 2, n - 1]) for s, t, n in zip(slots, seqs, lens)]).cpu().numpy()
    for j in range(len(slots)):
        assert rel_err(first[2 * j:2 * j + 2], want[j][:2]) <= tol, (what, "prompt", j)
    for i in range(FAR_DECODE):          # the first two steps run as they are, the others are a replayed recording
        out = eng.step([Entry(s, [t[n + i]], [0]) for s, t, n in zip(slots, seqs, lens)]).cpu().numpy()
        for j in range(len(slots)):
            assert rel_err(out[j], want[j][2 + i]) <= tol, (what, "token", i, "sequence", j)
    assert len(slots) in eng._graphs, "the last steps were meant to be replayed"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_sequence_of_twenty_thousand_tokens(far, dtype):
    folder, seqs, want = far
    tol = 5e-5 if dtype == "float32" else TOL[dtype]
    eng = engine_for(folder, dtype, max_tokens=20480, max_ctx=24576, max_step_tokens=2048)     # the prompt goes in ten pieces
    slots = eng.open(1)
    _prompt_then_tokens(eng, slots, seqs[:1], FAR_LENS[:1], want[:1], tol, dtype)
    assert eng.length(slots[0]) == 20000 + FAR_DECODE and len(eng.cache.held_pages(slots[0])) == 313
    eng.close(slots)
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_lengths_from_a_hundred_to_twenty_thousand(far, dtype):
    """One launch serves sequences that hold 2 pages and 313: each uses as many of the grid's blocks as its own pages
    call for.  The sequences are given in an order that is not the order of their lengths."""
    folder, seqs, want = far
    tol = 5e-5 if dtype == "float32" else TOL[dtype]
    held = sum((n + FAR_DECODE + 63) // 64 * 64 for n in FAR_LENS)
    eng = engine_for(folder, dtype, max_tokens=held, max_ctx=32768, max_step_tokens=4096, max_slots=8)
    order = [3, 0, 7, 1, 5, 2, 6, 4]
    slots = eng.open(8)
    pick = lambda xs: [xs[i] for i in order]
    _prompt_then_tokens(eng, slots, pick(seqs), pick(FAR_LENS), pick(want), tol, dtype)
    assert eng.free_pages() == (0,)
    eng.close(slots)
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_more_sequences_than_a_recorded_step_takes(folders, oracle, dtype):
    """150 sequences that start together and go on one token at a time: more than the largest batch for which single
    tokens are recorded and replayed, so each step goes in several runs; a few of them checked against the plain one."""
    from dlgo_amd.engine import Entry
    n = 150
    eng = engine_for(folders["A", dtype], dtype, max_tokens=n * 64, max_slots=n, graph_max_batch=64)
    rng = np.random.default_rng(8)
    seqs = [rng.integers(0, TINY_A["vocab_size"], size=int(rng.integers(1, 6)) + 4).tolist() for _ in range(n)]
    slots = eng.open(n)
    got = [[] for _ in range(n)]
    out = eng.step([Entry(s, t[:-4], [len(t) - 5]) for s, t in zip(slots, seqs)]).cpu().numpy()
    for i in range(n):
        got[i].append(out[i])
    for k in range(4, 0, -1):
        out = eng.step([Entry(s, [t[-k]], [0]) for s, t in zip(slots, seqs)]).cpu().numpy()
        for i in range(n):
            got[i].append(out[i].copy())
    for i in (0, 1, 63, 64, 65, 127, 128, 149):
        want = oracle("A", dtype, seqs[i])[len(seqs[i]) - 5:]
        assert rel_err(np.stack(got[i]), want) <= TOL[dtype], i
    eng.close(slots)
    eng.cache.check_consistent()


def test_errors_before_anything_runs(folders):
    from dlgo_amd.engine import EngineError, Entry
    eng = engine_for(folders["A", "float32"], "float32", max_tokens=128)
    (slot,) = eng.open(1)
    with pytest.raises(EngineError, match="vocabulary"):
        eng.step([Entry(slot, [1, 256], [0])])
    with pytest.raises(EngineError, match="no tokens"):
        eng.step([Entry(slot, [], [])])
    with pytest.raises(EngineError, match="twice"):
        eng.step([Entry(slot, [1], []), Entry(slot, [2], [])])
    with pytest.raises(EngineError, match="context"):
        eng.step([Entry(slot, [1] * 129, [])])
    with pytest.raises(EngineError, match="place"):
        eng.step([Entry(slot, [1, 2], [2])])
    with pytest.raises(EngineError):
        eng.step([Entry(99, [1], [])])
    assert eng.length(slot) == 0
    eng.step([Entry(slot, [1, 2, 3], [])])
    assert eng.length(slot) == 3


def test_a_decode_call_is_checked_whole_before_any_of_its_runs(folders):
    """More sequences than a recorded step's fixed arrays hold go in runs of that many; what is wrong with the call (a
    slot named in two different runs, a token outside the vocabulary in the last run, a sequence at the end of the
    context) is found before the first run has advanced anything."""
    from dlgo_amd.engine import EngineError, Entry
    eng = engine_for(folders["A", "float32"], "float32", max_tokens=1024, graph_max_batch=2)
    slots = eng.open(5)
    eng.step([Entry(s, [3, 4, 5], []) for s in slots])
    lengths = lambda: [eng.length(s) for s in slots]
    with pytest.raises(EngineError, match="distinct"):
        eng.decode([slots[0], slots[1], slots[2], slots[0]], [1, 2, 3, 4])       # twice, but once in each run of two
    assert lengths() == [3] * 5
    with pytest.raises(EngineError, match="vocabulary"):
        eng.decode(slots, [1, 2, 3, 4, 256])
    assert lengths() == [3] * 5
    with pytest.raises(EngineError, match="in use"):
        eng.decode(slots[:4] + [77], [1, 2, 3, 4, 5])
    assert lengths() == [3] * 5
    out = eng.decode(slots, [1, 2, 3, 4, 5])
    assert out.shape == (5, 256) and lengths() == [4] * 5
    eng.close(slots)
    eng.cache.check_consistent()


def test_fork_reports_what_it_cannot_do_as_the_engine_does(folders):
    from dlgo_amd.engine import EngineError, Entry
    eng = engine_for(folders["A", "float32"], "float32", max_tokens=3 * 64, max_slots=2)
    (a,) = eng.open(1)
    eng.step([Entry(a, list(range(70)), [])])                    # two of the three pages
    with pytest.raises(EngineError, match="fork: .*pages"):
        eng.fork(a)                                              # the copy would need two more
    b = eng.fork(a, 10)                                          # one page: fits
    with pytest.raises(EngineError, match="fork: .*no free slot"):
        eng.fork(a, 5)
    with pytest.raises(EngineError, match="fork: .*holds 70 tokens"):
        eng.close([b])
        eng.fork(a, 71)
    with pytest.raises(EngineError, match="fork: .*not in use"):
        eng.fork(b)
    eng.close([a])
    eng.cache.check_consistent()
    assert eng.free_slots() == 2 and eng.free_pages() == (3,)


def test_sizes_the_kernels_cannot_take_are_refused_at_once(tmp_path):
    """A width that is no multiple of the products' 16-byte loads: a clear error when the engine is made, for the
    dtype it concerns, not a wrong result later."""
    from dlgo_amd.engine import Engine, EngineError
    raw = dict(TINY_A, hidden_size=68, num_attention_heads=4, head_dim=16, intermediate_size=100)
    folder = make_folder(raw, 1, tmp_path, dtype="float32")
    with pytest.raises(EngineError, match="multiple of 8"):
        Engine.from_folder(folder, "bfloat16", max_tokens=128)
    big_head = make_folder(dict(TINY_A, hidden_size=64, num_attention_heads=1, num_key_value_heads=1, head_dim=528), 1,
                           tmp_path / "big_head", dtype="float32")
    with pytest.raises(EngineError, match="head size 528"):
        Engine.from_folder(big_head, "float32", max_tokens=128)
    eng = Engine.from_folder(folder, "float32", max_tokens=128)       # 68 and 100 are multiples of 4: float32 runs
    from dlgo_amd.engine import Entry
    (slot,) = eng.open(1)
    tokens = [3, 9, 27, 81]
    got = eng.step([Entry(slot, tokens, [0, 1, 2, 3])]).cpu().numpy()
    cfg, w = plain.read_model(folder)
    assert rel_err(got, plain.forward(cfg, w, tokens)) <= TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wanted_places_in_any_order_with_an_odd_vocabulary(folders, oracle, dtype):
    """Logits only where they are wanted, in the order asked, from a step that is cut into pieces; the vocabulary of
    this configuration (515) makes most rows of the output start at unaligned addresses."""
    from dlgo_amd.engine import Entry
    seqs = prompts_for(TINY_C, [90, 41, 7], seed=12)
    eng = engine_for(folders["C", dtype], dtype, max_step_tokens=32)
    slots = eng.open(3)
    wants = [[89, 0, 40], [], [6, 5]]
    out = eng.step([Entry(s, t, w) for s, t, w in zip(slots, seqs, wants)]).cpu().numpy()
    assert out.shape == (5, 515)
    rows = [(0, 89), (0, 0), (0, 40), (2, 6), (2, 5)]
    for r, (i, p) in enumerate(rows):
        assert rel_err(out[r], oracle("C", dtype, seqs[i])[p]) <= TOL[dtype], (r, i, p)
    assert [eng.length(s) for s in slots] == [90, 41, 7]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_model_with_attention_biases(tmp_path, dtype):
    """config.json's attention_bias: the four attention projections have a bias each.  Whole, in a batch of unequal
    lengths, and the last tokens one by one (a recorded step included), against the plain implementation."""
    from dlgo_amd.engine import Engine, Entry
    raw = dict(TINY_B, attention_bias=True)
    folder = make_folder(raw, 17, tmp_path, dtype=dtype, std=0.08, norm_jitter=0.1)
    cfg, w = plain.read_model(folder)
    assert "model.layers.2.self_attn.o_proj.bias" in w
    seqs = prompts_for(raw, [70, 9, 33], seed=12)
    want = [plain.forward(cfg, w, t) for t in seqs]
    # the biases matter: without them the logits are far away
    stripped = {k: v for k, v in w.items() if not k.endswith(".bias")}
    assert rel_err(plain.forward(cfg, stripped, seqs[1]), want[1]) > 5 * TOL[dtype]
    eng = Engine.from_folder(folder, dtype, max_tokens=1024)
    slots = eng.open(3)
    out = eng.step([Entry(s, t, list(range(len(t)))) for s, t in zip(slots, seqs)]).cpu().numpy()
    o = 0
    for t, wnt in zip(seqs, want):
        assert rel_err(out[o:o + len(t)], wnt) <= TOL[dtype]
        o += len(t)
    eng.close(slots)
    (slot,) = eng.open(1)
    rows = [eng.step([Entry(slot, seqs[0][:60], list(range(60)))])]
    for t in seqs[0][60:]:
        rows.append(eng.step([Entry(slot, [t], [0])]))
    assert rel_err(np.concatenate([r.cpu().numpy() for r in rows]), want[0]) <= TOL[dtype]
    assert 1 in eng._graphs
    eng.close([slot])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_steps_of_a_shape_seen_before_are_replayed(folders, oracle, dtype):
    """A step of fresh prompts is recorded the second time its shape (rows per sequence, wanted places) comes and replayed
    afterwards.  Every run of the shape, with other token ids each time and with other steps, other shapes and waits
    for the device between them, gives the plain logits; only two shapes are kept, so a third pushes the oldest out."""
    from dlgo_amd.engine import Entry
    raw = CONFIGS["B"][0]
    eng = engine_for(folders["B", dtype], dtype, max_tokens=4096, prompt_graph_limit=2)
    shapes = {"x": [17, 3, 40, 1], "y": [5], "z": [64, 65]}

    def run(name, seed):
        seqs = prompts_for(raw, shapes[name], seed=seed)
        slots = eng.open(len(seqs))
        got = eng.step([Entry(s, t, [0, len(t) - 1] if len(t) > 1 else [0]) for s, t in zip(slots, seqs)])
        # decoding goes on from a replayed prompt as from any other: one more token for the first sequence
        more = eng.step([Entry(slots[0], [7], [0])])
        torch.cuda.synchronize()
        got, more = got.cpu().numpy(), more.cpu().numpy()
        row = 0
        for t in seqs:
            want = oracle("B", dtype, t)
            for place in ([0, len(t) - 1] if len(t) > 1 else [0]):
                assert rel_err(got[row], want[place]) <= TOL[dtype], (name, seed, len(t), place)
                row += 1
        assert rel_err(more[0], oracle("B", dtype, seqs[0] + [7])[-1]) <= TOL[dtype], (name, seed)
        eng.close(slots)

    order = [("x", 1), ("y", 2), ("x", 3), ("x", 4), ("y", 5), ("z", 6), ("y", 7), ("z", 8), ("x", 9), ("x", 10), ("z", 11)]
    for name, seed in order:
        run(name, seed)
    recorded = {len(k[0]) for k in eng._prompt_graphs}
    assert len(eng._prompt_graphs) == 2 and recorded <= {4, 1, 2}
    eng.cache.check_consistent()
    # the same with recording switched off gives the same numbers
    plain_eng = engine_for(folders["B", dtype], dtype, max_tokens=4096, use_graphs=False)
    seqs = prompts_for(raw, shapes["x"], seed=3)
    for e in (eng, plain_eng):
        slots = e.open(4)
        e.last = e.step([Entry(s, t, [len(t) - 1]) for s, t in zip(slots, seqs)]).cpu().numpy()
        e.close(slots)
    slots = eng.open(4)
    again = eng.step([Entry(s, t, [len(t) - 1]) for s, t in zip(slots, seqs)]).cpu().numpy()     # replayed now
    eng.close(slots)
    assert np.array_equal(again, plain_eng.last) and np.array_equal(eng.last, plain_eng.last)
