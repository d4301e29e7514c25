"""Generation through the entry point, the command line and the replay program, on the GPU."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import plain_llama as plain
from conftest import ROOT, TINY_A, TINY_B, make_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folder_a(tmp_path_factory):
    return make_folder(TINY_A, 21, tmp_path_factory.mktemp("gen_a"), dtype="float32", std=0.1)


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory):
    return make_folder(TINY_B, 22, tmp_path_factory.mktemp("gen_b"), dtype="float32", std=0.08, norm_jitter=0.1)


def _prompts(raw, lens, seed):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, raw["vocab_size"], size=n).tolist() for n in lens]


def test_greedy_matches_plain_in_unequal_batches(folder_a):
    """Tiny A's workload: prompts of 5, 9 and 1 tokens, 8 tokens each, then more requests than fit at once."""
    import dlgo_amd
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="float32", max_tokens=512, max_batch=3)
    prompts = _prompts(TINY_A, [5, 9, 1, 12, 3, 30, 2], seed=1)
    streamed = []
    results = llm.generate(prompts, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(8), dlgo_amd.with_ignore_eos())
    for p, r in zip(prompts, results):
        assert r.tokens == plain.greedy_generate(cfg, w, p, 8)
        assert r.finish_reason == "length"
    llm.engine.cache.check_consistent()
    assert llm.engine.free_slots() == llm.engine.cache.max_slots
    r = llm.generate_stream(prompts[0], streamed.append, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(8),
                            dlgo_amd.with_ignore_eos())
    assert streamed == r.tokens == results[0].tokens          # one call per token, same tokens alone as in a batch


def test_stop_tokens_end_sequences_early(folder_a):
    import dlgo_amd
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="float32", max_tokens=512)
    prompts = _prompts(TINY_A, [4, 7, 2], seed=2)
    free = [plain.greedy_generate(cfg, w, p, 10) for p in prompts]
    stop = free[1][3]
    results = llm.generate(prompts, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(10), dlgo_amd.with_stop_tokens([stop]))
    for p, r in zip(prompts, results):
        want = plain.greedy_generate(cfg, w, p, 10, stop_tokens=(stop,))
        assert r.tokens == want
        assert r.finish_reason == ("stop" if len(want) < 10 else "length")
    assert results[1].finish_reason == "stop" and stop not in results[1].tokens


def test_temperature_sampling_is_reproducible_and_matches_plain(folder_b):
    """Tiny B's workload: prompts 17, 3, 40, 1; 12 tokens at temperature 0.8 with a fixed seed, beside a greedy run."""
    import dlgo_amd
    from dlgo_amd.sampling import uniform
    cfg, w = plain.read_model(folder_b)
    llm = dlgo_amd.load_llm(folder_b, dtype="float32", max_tokens=1024)
    prompts = _prompts(TINY_B, [17, 3, 40, 1], seed=3)
    opts = [dlgo_amd.with_temperature(0.8), dlgo_amd.with_top_k(0), dlgo_amd.with_top_p(1.0), dlgo_amd.with_repetition_penalty(1.0),
            dlgo_amd.with_seed(1234), dlgo_amd.with_max_tokens(12), dlgo_amd.with_ignore_eos()]
    a = llm.generate(prompts, *opts)
    b = llm.generate(prompts, *opts)
    assert [r.tokens for r in a] == [r.tokens for r in b]
    alone = llm.generate([prompts[2]], *opts)
    # a request's draws are keyed by its index in the call, so alone (index 0) it draws differently from index 2
    assert len(alone[0].tokens) == 12
    for i, (p, r) in enumerate(zip(prompts, a)):
        seq, want = list(p), []
        for step in range(12):
            tok = plain.sample_token(plain.forward(cfg, w, seq)[-1], uniform(1234, i, step), 0.8)
            want.append(tok)
            seq.append(tok)
        assert r.tokens == want, i
    g = llm.generate(prompts, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(12), dlgo_amd.with_ignore_eos())
    for p, r in zip(prompts, g):
        assert r.tokens == plain.greedy_generate(cfg, w, p, 12)
    # dlgo's default sampler (temperature 0.7, top-k 40, top-p 0.9, penalty 1.1) runs and respects the seed
    d1 = llm.generate(prompts, dlgo_amd.with_seed(5), dlgo_amd.with_max_tokens(12))
    d2 = llm.generate(prompts, dlgo_amd.with_seed(5), dlgo_amd.with_max_tokens(12))
    assert [r.tokens for r in d1] == [r.tokens for r in d2]
    # ... and draws what the plain pipeline draws, the penalty looking back on the tokens generated so far; two
    # requests at a time, so that the second pair takes over the first pair's slots and must not inherit their tokens
    small = dlgo_amd.load_llm(folder_b, dtype="float32", max_tokens=1024, max_batch=2)
    d3 = small.generate(prompts, dlgo_amd.with_seed(5), dlgo_amd.with_max_tokens(12), dlgo_amd.with_ignore_eos())
    for i, (p, r) in enumerate(zip(prompts, d3)):
        seq, want = list(p), []
        for step in range(12):
            tok = plain.sample_token(plain.forward(cfg, w, seq)[-1], uniform(5, i, step), 0.7, 40, 0.9, 0.0, 1.1, want[-64:])
            want.append(tok)
            seq.append(tok)
        assert r.tokens == want, i


def test_long_decoding_and_context_end(folder_a):
    """Decoding up to the end of the context: the last tokens still match, and the run ends with "context"."""
    import dlgo_amd
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="float32", max_tokens=512)
    prompt = _prompts(TINY_A, [3], seed=4)[0]
    r = llm.generate(prompt, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(500), dlgo_amd.with_ignore_eos())
    assert r.finish_reason == "context"
    assert len(prompt) + len(r.tokens) == TINY_A["max_position_embeddings"] - 1
    assert r.tokens == plain.greedy_generate(cfg, w, prompt, len(r.tokens))
    with pytest.raises(ValueError, match="prompt too long"):
        llm.generate([1] * 128, dlgo_amd.with_greedy())


def _check_against_margin(cfg, w, prompt, tokens, tol):
    """Greedy tokens of a reduced-precision run, against the plain logits of the same sequence: where the plain
    implementation's best token leads by more than the run's error bound the run must have chosen it, elsewhere a
    token within the bound of the best."""
    seq = list(prompt)
    decided = 0
    for tok in tokens:
        logits = plain.forward(cfg, w, seq)[-1]
        bound = 2.0 * tol * np.abs(logits).max()
        best = int(np.argmax(logits))
        if logits[best] - np.partition(logits, -2)[-2] > bound:
            assert tok == best, (len(seq), tok, best)
            decided += 1
        else:
            assert logits[tok] >= logits[best] - bound, (len(seq), tok, best)
        seq.append(tok)
    return decided


def test_bfloat16_generation_follows_the_plain_logits_where_their_margin_allows(folder_a):
    import dlgo_amd
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="bfloat16", max_tokens=512)
    prompts = _prompts(TINY_A, [5, 9, 1, 30], seed=7)
    results = llm.generate(prompts, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(24), dlgo_amd.with_ignore_eos())
    decided = sum(_check_against_margin(cfg, w, p, r.tokens, 3e-2) for p, r in zip(prompts, results))
    assert all(len(r.tokens) == 24 for r in results)
    assert decided >= 48, "too few tokens had a margin: the check says little"      # most steps of this model are clear


def test_the_repetition_penalty_looks_back_64_tokens_also_after_the_ring_wraps(folder_a):
    """More than 64 generated tokens with a penalty: the device's ring of recent tokens wraps, and every choice still is
    the plain pipeline's over the last 64 tokens."""
    import dlgo_amd
    from dlgo_amd.sampling import uniform
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="float32", max_tokens=512, max_batch=2)
    prompts = _prompts(TINY_A, [4, 11, 2], seed=8)
    n = 90
    opts = [dlgo_amd.with_temperature(0.9), dlgo_amd.with_top_k(0), dlgo_amd.with_top_p(1.0), dlgo_amd.with_repetition_penalty(1.5),
            dlgo_amd.with_seed(77), dlgo_amd.with_max_tokens(n), dlgo_amd.with_ignore_eos()]
    results = llm.generate(prompts, *opts)
    for i, (p, r) in enumerate(zip(prompts, results)):
        seq, want = list(p), []
        for step in range(n):
            tok = plain.sample_token(plain.forward(cfg, w, seq)[-1], uniform(77, i, step), 0.9, 0, 1.0, 0.0, 1.5, want[-64:])
            want.append(tok)
            seq.append(tok)
        assert r.tokens == want, i
        # the window matters here: with the whole history penalised the run would differ
        seq, other = list(p), []
        for step in range(n):
            tok = plain.sample_token(plain.forward(cfg, w, seq)[-1], uniform(77, i, step), 0.9, 0, 1.0, 0.0, 1.5, other)
            other.append(tok)
            seq.append(tok)
        if i == 0:
            assert other != want


@pytest.mark.parametrize("options", [dict(graph_max_batch=4), dict(max_step_tokens=3), dict(use_graphs=False)])
def test_more_sequences_than_a_recorded_step_holds(folder_a, options):
    """Seven sequences decode together where a recorded step has fixed arrays for four (or the workspace rows for
    three): the step runs in several runs and generation gives the plain tokens."""
    import dlgo_amd
    cfg, w = plain.read_model(folder_a)
    llm = dlgo_amd.load_llm(folder_a, dtype="float32", max_tokens=1024, max_batch=7, **options)
    prompts = _prompts(TINY_A, [5, 9, 1, 12, 3, 30, 2], seed=9)
    results = llm.generate(prompts, dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(6), dlgo_amd.with_ignore_eos())
    for p, r in zip(prompts, results):
        assert r.tokens == plain.greedy_generate(cfg, w, p, 6)
    assert llm.engine.free_slots() == llm.engine.cache.max_slots
    b = llm.benchmark(prompts[0], dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(6), dlgo_amd.with_ignore_eos())
    assert b.tokens == results[0].tokens and len(b.step_ms) == 1 + 6 and b.total_ms >= b.prefill_ms + b.generate_ms - 1e-3
    assert b.architecture == "LlamaForCausalLM" and b.output_tokens == 6 and b.prompt_tokens == 5


def test_command_line(folder_a):
    out = subprocess.run([sys.executable, "-m", "dlgo_amd", "--greedy", "--max-tokens", "4", "--dtype", "float32", "--ignore-eos",
                          "--prompt-ids", "5,6,7", "--prompt-ids", "9", folder_a], cwd=ROOT, capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stderr
    cfg, w = plain.read_model(folder_a)
    lines = [json.loads(l) for l in out.stdout.splitlines() if l.startswith("{")]
    assert lines[0]["tokens"] == plain.greedy_generate(cfg, w, [5, 6, 7], 4)
    assert lines[1]["tokens"] == plain.greedy_generate(cfg, w, [9], 4)
    bad = subprocess.run([sys.executable, "-m", "dlgo_amd", "--temp", "-1", folder_a], cwd=ROOT, capture_output=True, text=True)
    assert bad.returncode == 1 and "--temp must be >= 0" in bad.stderr


def test_a_model_from_a_configuration_and_a_seed_without_any_file(tmp_path):
    """load_llm, the command line and the replay program run a model whose weights are drawn for a seed; the plain side
    computes the same weights itself (its own generator, element by element) and gives the same tokens and logits."""
    import dlgo_amd
    from dlgo_amd.config import config_from_dict
    raw = dict(TINY_B, initializer_range=0.09)
    w = plain.random_model(raw, 33)
    prompts = _prompts(TINY_B, [6, 2, 11], seed=12)
    want = [plain.greedy_generate(raw, w, p, 5) for p in prompts]
    opts = (dlgo_amd.with_greedy(), dlgo_amd.with_max_tokens(5), dlgo_amd.with_ignore_eos())
    cfg_file = tmp_path / "b.json"
    cfg_file.write_text(json.dumps(raw))
    for source in (raw, config_from_dict(raw), str(cfg_file)):
        llm = dlgo_amd.load_llm(source, dtype="float32", max_tokens=512, random_seed=33)
        assert [r.tokens for r in llm.generate(prompts, *opts)] == want
    assert [r.tokens for r in dlgo_amd.load_llm(raw, dtype="float32", max_tokens=512, random_seed=34).generate(prompts, *opts)] != want
    with pytest.raises(Exception, match="random_seed"):
        dlgo_amd.load_llm(raw, dtype="float32", max_tokens=512)
    # the command line
    out = subprocess.run([sys.executable, "-m", "dlgo_amd", "--random-config", str(cfg_file), "--weight-seed", "33", "--greedy",
                          "--max-tokens", "5", "--dtype", "float32", "--ignore-eos"] +
                         [a for p in prompts for a in ("--prompt-ids", ",".join(map(str, p)))],
                         cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert [json.loads(l)["tokens"] for l in out.stdout.splitlines() if l.startswith("{")] == want
    both = subprocess.run([sys.executable, "-m", "dlgo_amd", "--random-config", str(cfg_file), str(tmp_path)], cwd=ROOT,
                          capture_output=True, text=True)
    assert both.returncode == 2 and "one of them" in both.stderr
    # the replay program
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": prompts[2], "want": list(range(len(prompts[2])))}], "end": ["x"]}]
    text = "".join(json.dumps(s_) + "\n" for s_ in steps)
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--config", str(cfg_file), "--weight-seed", "33", "--dtype", "float32",
                        "--out", str(tmp_path / "out"), "--max-tokens", "64"], input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0 and "done 0" in p.stdout, p.stderr
    got = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(-1, TINY_B["vocab_size"])
    ref = plain.forward(raw, w, prompts[2])
    assert np.abs(got - ref).max() <= 2e-5 * np.abs(ref).max()
    assert json.load(open(tmp_path / "out" / "index.json"))["weight_seed"] == 33


def _replay(folder, dtype, steps, out_dir, max_tokens):
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out_dir),
                        "--max-tokens", str(max_tokens)], input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay(folder_b, tmp_path, dtype):
    cfg, w = plain.read_model(folder_b)
    V = TINY_B["vocab_size"]
    seqs = dict(zip("abcd", _prompts(TINY_B, [70, 40, 9, 100], seed=6)))
    want = {k: plain.forward(cfg, w, v) for k, v in seqs.items()}
    tol = 2e-5 if dtype == "float32" else 3e-2
    # whole
    steps = [{"step": i, "entries": [{"id": k, "tokens": v, "want": list(range(len(v)))}], "end": [k]}
             for i, (k, v) in enumerate(seqs.items())]
    _replay(folder_b, dtype, steps, tmp_path / "whole", 128)
    index = json.load(open(tmp_path / "whole" / "index.json"))
    assert index["vocab"] == V and index["dtype"] == dtype and sorted(index["steps"]) == ["0", "1", "2", "3"]
    assert index["steps"]["2"] == {"file": "2.f32", "shape": [9, V], "rows": [["c", i] for i in range(9)]}
    for i, k in enumerate(seqs):
        got = np.fromfile(tmp_path / "whole" / f"{i}.f32", dtype="<f4").reshape(-1, V)
        assert np.abs(got - want[k]).max() <= tol * np.abs(want[k]).max()
    # the last 32 one by one
    v = seqs["d"]
    head = len(v) - 32
    steps = [{"step": 0, "entries": [{"id": "d", "tokens": v[:head], "want": [0, head - 1]}], "end": []}]
    steps += [{"step": 1 + i, "entries": [{"id": "d", "tokens": [t], "want": [0]}], "end": ["d"] if i == 31 else []}
              for i, t in enumerate(v[head:])]
    _replay(folder_b, dtype, steps, tmp_path / "tail", 128)
    got = np.fromfile(tmp_path / "tail" / "0.f32", dtype="<f4").reshape(-1, V)
    assert np.abs(got - want["d"][[0, head - 1]]).max() <= tol * np.abs(want["d"]).max()
    for i in range(32):
        got = np.fromfile(tmp_path / "tail" / f"{1 + i}.f32", dtype="<f4").reshape(-1, V)
        assert np.abs(got[0] - want["d"][head + i]).max() <= tol * np.abs(want["d"]).max()
    # a batch of unequal lengths whose shorter requests end earlier, then another in the same room
    first = {"a": 60, "b": 35, "c": 1}
    steps = [{"step": 0, "entries": [{"id": k, "tokens": seqs[k][:p], "want": [p - 1]} for k, p in first.items()], "end": []}]
    n = 1
    pos = dict(first)
    while any(pos[k] < len(seqs[k]) for k in first):
        live = [k for k in first if pos[k] < len(seqs[k])]
        ends = [k for k in live if pos[k] + 1 == len(seqs[k])]
        steps.append({"step": n, "entries": [{"id": k, "tokens": [seqs[k][pos[k]]], "want": [0]} for k in live], "end": ends})
        for k in live:
            pos[k] += 1
        n += 1
    steps.append({"step": n, "entries": [{"id": "d", "tokens": seqs["d"], "want": [99]}], "end": ["d"]})
    _replay(folder_b, dtype, steps, tmp_path / "batch", 256)
    index = json.load(open(tmp_path / "batch" / "index.json"))
    assert index["steps"]["0"]["rows"] == [["a", 59], ["b", 34], ["c", 0]] and index["steps"]["0"]["shape"] == [3, V]
    assert len(index["steps"]) == len(steps)
    got0 = np.fromfile(tmp_path / "batch" / "0.f32", dtype="<f4").reshape(-1, V)
    for r, (k, p) in enumerate(first.items()):
        assert np.abs(got0[r] - want[k][p - 1]).max() <= tol * np.abs(want[k]).max()
    pos = dict(first)
    for s in steps[1:-1]:
        got = np.fromfile(tmp_path / "batch" / f"{s['step']}.f32", dtype="<f4").reshape(-1, V)
        for r, e in enumerate(s["entries"]):
            k = e["id"]
            assert np.abs(got[r] - want[k][pos[k]]).max() <= tol * np.abs(want[k]).max(), (s["step"], k)
            pos[k] += 1
    got = np.fromfile(tmp_path / "batch" / f"{n}.f32", dtype="<f4").reshape(-1, V)
    assert np.abs(got[0] - want["d"][99]).max() <= tol * np.abs(want["d"]).max()
