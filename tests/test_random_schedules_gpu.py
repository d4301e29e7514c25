"""Seeded random configurations of the architecture and random ways of cutting requests into steps, against the plain
implementation: prompts in two pieces of random sizes with batch mates of other lengths, then the last tokens one by
one, some requests leaving early, a second batch on the slots of the first.  The sizes are drawn so that grids of
blocks get shapes the fixed tests do not have (many heads to a kv head, many sequences, rows of tiles that do not
divide the chip); the first two cases once computed a sequence's tiles twice or not at all."""
import numpy as np
import pytest

import plain_llama as plain
from conftest import make_folder

pytestmark = pytest.mark.gpu

TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def draw_config(rng):
    kv, group = int(rng.choice([1, 2, 3, 4])), int(rng.choice([1, 2, 3, 4, 5, 8]))
    raw = {"architectures": ["LlamaForCausalLM"], "vocab_size": int(rng.choice([97, 256, 1000, 1531])),
           "hidden_size": int(rng.choice([64, 72, 136, 200, 256, 320])), "num_hidden_layers": int(rng.choice([1, 2, 3])),
           "intermediate_size": int(rng.choice([64, 104, 264, 512])), "num_attention_heads": kv * group,
           "num_key_value_heads": kv, "head_dim": int(rng.choice([16, 32, 48, 64, 80, 128])),
           "rms_norm_eps": float(rng.choice([1e-5, 1e-6])), "rope_theta": float(rng.choice([10000.0, 500000.0])),
           "max_position_embeddings": 1024, "tie_word_embeddings": bool(rng.integers(2)), "initializer_range": 0.05}
    if rng.integers(2):
        raw["rope_scaling"] = {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                               "original_max_position_embeddings": 64}
    return raw


def run_schedule(eng, cfg, weights, vocab, rng, batches):
    """The largest error, relative to the largest logit of a request, over everything the schedule computes."""
    from dlgo_amd.engine import Entry
    worst = 0.0
    for lens in batches:
        k = len(lens)
        seqs = [rng.integers(0, vocab, size=n).tolist() for n in lens]
        want = [plain.forward(cfg, weights, s) for s in seqs]
        tail = [int(min(n - 1, rng.integers(0, 6))) for n in lens]                  # tokens that come one by one
        cut = [int(rng.integers(1, n - t + 1)) if n - t > 1 else n - t for n, t in zip(lens, tail)]
        slots = list(eng.open(k))
        got = [np.full_like(x, np.nan) for x in want]
        done = [0] * k

        def run(pieces):
            entries, places = [], []
            for i, n in pieces:
                if n > 0:
                    entries.append(Entry(slots[i], seqs[i][done[i]:done[i] + n], list(range(n))))
                    places.append((i, done[i], n))
            if not entries:
                return
            out = eng.step(entries).cpu().numpy()
            r = 0
            for i, p0, n in places:
                got[i][p0:p0 + n] = out[r:r + n]
                r += n
                done[i] += n
        run([(i, cut[i]) for i in range(k)])
        run([(i, lens[i] - tail[i] - done[i]) for i in range(k)])
        while any(done[i] < lens[i] for i in range(k)):
            run([(i, 1) for i in range(k) if done[i] < lens[i]])
            for i in range(k):
                if done[i] == lens[i] and slots[i] is not None and rng.integers(2):
                    eng.close([slots[i]])                                           # some leave early: the slot goes back
                    slots[i] = None
        eng.close([s for s in slots if s is not None])
        for a, b in zip(got, want):
            worst = max(worst, float(np.abs(a - b).max() / np.abs(b).max()))
    return worst


FIXED = [   # (heads, kv heads, head size, batches of request lengths)
    (32, 4, 128, [[65, 63, 17, 1], [63, 300, 2, 300, 2]]),
    (32, 4, 32, [[63], [300, 65, 64, 64]]),
    (24, 8, 128, [[700, 650, 64, 300, 641, 90]]),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", range(len(FIXED) + 8))
def test_random_schedule(tmp_path, case, dtype):
    from dlgo_amd.engine import Engine
    rng = np.random.default_rng(7000 + case)
    raw = draw_config(rng)
    if case < len(FIXED):
        heads, kv, hd, batches = FIXED[case]
        raw.update(num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, num_hidden_layers=1)
    else:
        batches = [[int(rng.choice([1, 2, 17, 63, 64, 65, 130, 300])) for _ in range(int(rng.integers(1, 6)))] for _ in range(2)]
    folder = make_folder(raw, int(rng.integers(100)), tmp_path, dtype, norm_jitter=0.1)
    cfg, weights = plain.read_model(str(folder))
    eng = Engine.from_folder(str(folder), dtype, max_tokens=4096, max_step_tokens=int(rng.choice([64, 200, 4096])))
    err = run_schedule(eng, cfg, weights, raw["vocab_size"], rng, batches)
    assert err <= TOL[dtype], (raw, batches, err)
