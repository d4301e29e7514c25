"""Real layer sizes with one or two layers: whole, the last 32 tokens one by one, batches of unequal lengths one after the
other in reused slots and pages, and the benchmark's decode shapes, against the plain implementation, in float32 and bfloat16.

  1b: Llama 3.2 1B (hidden 2048, 32 heads over 8 kv heads of 64, feed-forward 8192, vocabulary 128256, scaling factor 32)
  3b: Llama 3.2 3B layers (hidden 3072, 24 heads over 8 kv heads of 128: three query heads a group, feed-forward 8192)
  8b: Llama 3.1 8B layers (hidden 4096, 32 heads over 8 kv heads of 128, feed-forward 14336, untied head, factor 8)
  wide: a hidden size of 5120 (40 heads over 8 kv heads of 128), wider than the streamed products' hand-off of a norm
        covers: its decode steps take the norm kernels instead
The larger ones have one layer and a vocabulary of 32003 to keep the plain implementation quick."""
import numpy as np
import pytest

import plain_llama as plain
from conftest import make_folder

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 128256, "hidden_size": 2048, "num_hidden_layers": 2, "intermediate_size": 8192,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "tie_word_embeddings": True, "initializer_range": 0.02,
    "hidden_act": "silu", "torch_dtype": "bfloat16",
}
WIDE_3B = dict(WIDE, vocab_size=32003, hidden_size=3072, num_hidden_layers=1, num_attention_heads=24, head_dim=128)
WIDE_8B = dict(WIDE, vocab_size=32003, hidden_size=4096, num_hidden_layers=1, intermediate_size=14336, head_dim=128,
               tie_word_embeddings=False,
               rope_scaling=dict(WIDE["rope_scaling"], factor=8.0))
WIDE_5120 = dict(WIDE_3B, hidden_size=5120, num_attention_heads=40, intermediate_size=6144)
SHAPES = {"1b": WIDE, "3b": WIDE_3B, "8b": WIDE_8B, "wide": WIDE_5120}


@pytest.fixture(scope="module")
def folder_1b(tmp_path_factory):
    return make_folder(WIDE, 31, tmp_path_factory.mktemp("wide_1b"), dtype="bfloat16")


@pytest.fixture(scope="module", params=list(SHAPES))
def wide(request, tmp_path_factory):
    raw = SHAPES[request.param]
    if request.param == "1b":
        folder = request.getfixturevalue("folder_1b")
    else:
        folder = make_folder(raw, 31, tmp_path_factory.mktemp("wide_" + request.param), dtype="bfloat16")
    cfg, w = plain.read_model(folder)
    rng = np.random.default_rng(2)
    seqs = [rng.integers(0, raw["vocab_size"], size=n).tolist() for n in (70, 9)]
    # positions far into the context, where the scaled low frequencies matter
    want = [plain.forward(cfg, w, s) for s in seqs]
    return folder, seqs, want


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 3e-2)])
def test_real_widths(wide, dtype, tol):
    from dlgo_amd.engine import Engine, Entry
    folder, seqs, want = wide
    eng = Engine.from_folder(folder, dtype, max_tokens=512)
    err = lambda got, ref: np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max()
    # whole, in one batch of unequal lengths
    slots = eng.open(2)
    out = eng.step([Entry(s, t, list(range(len(t)))) for s, t in zip(slots, seqs)]).cpu().numpy()
    assert err(out[:70], want[0]) <= tol and err(out[70:], want[1]) <= tol
    assert (out[:70].argmax(-1) == want[0].argmax(-1)).mean() >= (1.0 if dtype == "float32" else 0.9)
    eng.close(slots)
    # a prompt and then the last 32 tokens one by one: the first two steps run as they are, the rest as a replayed recording
    (slot,) = eng.open(1)
    got = [eng.step([Entry(slot, seqs[0][:38], list(range(38)))]).cpu().numpy()]
    for t in seqs[0][38:]:
        got.append(eng.step([Entry(slot, [t], [0])]).cpu().numpy().copy())
    assert err(np.concatenate(got), want[0]) <= tol
    assert 1 in eng._graphs
    eng.close([slot])


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 3e-2)])
def test_real_widths_batches_reuse_slots_and_pages(wide, dtype, tol):
    """Two batches of unequal lengths, one after the other, in a cache that holds exactly one of them: the second batch
    runs in the slots and pages the first gave back, with the sequences in the other order; its shorter request ends
    earlier (it stops after its prompt while the longer one goes on token by token)."""
    from dlgo_amd.engine import Engine, Entry
    folder, seqs, want = wide
    eng = Engine.from_folder(folder, dtype, max_tokens=192, max_slots=2)      # 70 -> two pages, 9 -> one
    err = lambda got, ref: np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max()
    assert eng.free_pages() == (3,)
    for order in ((0, 1), (1, 0)):
        slots = eng.open(2)
        assert eng.free_slots() == 0
        long_slot, short_slot = slots[order.index(0)], slots[order.index(1)]
        cut = 60                                            # the long one brings 60 tokens, then 10 more one by one
        entries = [None, None]
        entries[order.index(0)] = Entry(long_slot, seqs[0][:cut], list(range(cut)))
        entries[order.index(1)] = Entry(short_slot, seqs[1], list(range(len(seqs[1]))))
        out = eng.step(entries).cpu().numpy()
        a, b = (out[:cut], out[cut:]) if order == (0, 1) else (out[len(seqs[1]):], out[:len(seqs[1])])
        assert err(b, want[1]) <= tol
        eng.close([short_slot])                             # the shorter request ends; the longer one goes on alone
        got = [a]
        for t in seqs[0][cut:]:
            got.append(eng.step([Entry(long_slot, [t], [0])]).cpu().numpy().copy())
        assert err(np.concatenate(got), want[0]) <= tol
        eng.close([long_slot])
        assert eng.free_pages() == (3,) and eng.free_slots() == 2
        eng.cache.check_consistent()


# -- the benchmark's own decode shapes ------------------------------------------------------------------------------
# 1, 8 and 64 sequences of the 1B widths with 2,048 to 2,300 cached keys each, then four single-token steps: the first two
# run as they are, the third and fourth as a replayed recording.  At batch 8 the decode attention rotates and stores by
# itself and its pages are dealt to several blocks whose results a second kernel merges (at batch 1 to many more of
# them, and the products stream their weights against a single row); at batch 64 the rotation kernel
# reads the QKV product's unsummed runs and the 64x64 tiles do gate/up.  The plain implementation follows a few of the
# sequences (each whole, in float64); the first one has 2,048 tokens, so its first decoded token opens a new page.
BENCH_DECODE_STEPS = 4
_bench_plain = {}


def _bench_sequence(i):
    rng = np.random.default_rng(1000 + i)
    length = 2048 if i == 0 else 2048 + int(rng.integers(1, 252))
    return rng.integers(0, WIDE["vocab_size"], size=length + BENCH_DECODE_STEPS).tolist(), length


def _bench_plain_rows(folder, i):
    if i not in _bench_plain:
        if "model" not in _bench_plain:
            _bench_plain["model"] = plain.read_model(folder)
        cfg, w = _bench_plain["model"]
        tokens, length = _bench_sequence(i)
        _bench_plain[i] = plain.forward(cfg, w, tokens, rows=range(length - 1, length + BENCH_DECODE_STEPS))
    return _bench_plain[i]


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 3e-2)])
@pytest.mark.parametrize("batch,checked,max_ctx", [(1, (0,), 4096), (8, (0, 5), 4096), (64, (0, 5, 40), 4096),
                                                   # a recorded step is launched for the longest sequence the cache allows:
                                                   # of the blocks that a context of 32,768 gives a sequence, these use one
                                                   (64, (0, 5, 40), 32768)])
def test_benchmark_decode_shapes(folder_1b, batch, checked, max_ctx, dtype, tol):
    from dlgo_amd.engine import Engine, Entry
    seqs = [_bench_sequence(i) for i in range(batch)]
    eng = Engine.from_folder(folder_1b, dtype, max_tokens=batch * 2368, max_ctx=max_ctx)
    slots = eng.open(batch)
    rows = [eng.step([Entry(s, t[:n], [n - 1]) for s, (t, n) in zip(slots, seqs)]).cpu().numpy()]
    for k in range(BENCH_DECODE_STEPS):
        rows.append(eng.decode(slots, [t[n + k] for t, n in seqs]).cpu().numpy().copy())
    assert batch in eng._graphs, "the last steps were meant to be replayed"
    got = np.stack(rows, axis=1)                      # [sequence, step, vocabulary]
    assert np.isfinite(got).all()
    err = lambda g, ref: np.abs(g.astype(np.float64) - ref).max() / np.abs(ref).max()
    for i in checked:
        want = _bench_plain_rows(folder_1b, i)
        for k in range(BENCH_DECODE_STEPS + 1):
            assert err(got[i, k], want[k]) <= tol, (batch, dtype, i, k)
        if dtype == "float32":
            assert (got[i].argmax(-1) == want.argmax(-1)).all()
    eng.close(slots)
    eng.cache.check_consistent()


# -- sampling through the generation loop at the real vocabulary ----------------------------------------------------
def _draw_is_the_plain_one(logits, tok, u, slack, **options):
    """Whether `tok` is what the plain pipeline draws from these (plain) logits with the uniform u, give or take `slack`
    of cumulative probability: the engine's logits differ from the plain ones by rounding, and over 128,256 tokens the
    steps of the cumulative sum are as small as that difference.  Returns (exactly the plain token, within the slack)."""
    want = plain.sample_token(logits, u, **options)
    if tok == want:
        return True, True
    kept = plain.filtered_logits(logits, **options)
    if not np.isfinite(kept[tok]):
        return False, False
    cum = np.cumsum(plain.softmax(kept))
    below = cum[tok - 1] if tok > 0 else 0.0
    return False, below - slack <= u <= cum[tok] + slack


@pytest.mark.parametrize("options", [dict(temperature=0.8, top_k=0, top_p=1.0, penalty=1.0),
                                     dict(temperature=0.7, top_k=40, top_p=0.9, penalty=1.1)],      # the reference's defaults
                         ids=["temperature alone", "the default filters"])
def test_sampled_generation_at_the_real_vocabulary(folder_1b, options):
    """generate() with a temperature alone (a row of 128,256 that nothing cuts goes to 32 blocks and is drawn from their
    masses) and with the reference's default filters (top-k over 32 blocks), three requests of unequal lengths: every
    token is the one the plain pipeline draws from the plain logits of the same history with the same uniform number."""
    import dlgo_amd
    from dlgo_amd.sampling import uniform
    cfg, w = plain.read_model(folder_1b)
    llm = dlgo_amd.load_llm(folder_1b, dtype="float32", max_tokens=1024, max_batch=4)
    rng = np.random.default_rng(11)
    prompts = [rng.integers(0, WIDE["vocab_size"], size=n).tolist() for n in (9, 3, 14)]
    n_new = 5
    opts = [dlgo_amd.with_temperature(options["temperature"]), dlgo_amd.with_top_k(options["top_k"]),
            dlgo_amd.with_top_p(options["top_p"]), dlgo_amd.with_repetition_penalty(options["penalty"]), dlgo_amd.with_seed(99),
            dlgo_amd.with_max_tokens(n_new), dlgo_amd.with_ignore_eos()]
    results = llm.generate(prompts, *opts)
    again = llm.generate(prompts, *opts)
    assert [r.tokens for r in results] == [r.tokens for r in again]
    exact = total = 0
    for i, (p, r) in enumerate(zip(prompts, results)):
        assert len(r.tokens) == n_new
        seq = list(p)
        for step, tok in enumerate(r.tokens):
            logits = plain.forward(cfg, w, seq, rows=[len(seq) - 1])[0]
            same, near = _draw_is_the_plain_one(logits, tok, uniform(99, i, step), 3e-5, recent=r.tokens[:step][-64:], **options)
            assert near, (i, step, tok)
            exact += same
            total += 1
            seq.append(tok)
    assert exact >= 0.6 * total, f"only {exact} of {total} tokens are the plain ones exactly: the slack decides too often"
