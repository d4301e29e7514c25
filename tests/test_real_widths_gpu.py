"""Real layer sizes with one or two layers: whole, last tokens one by one, and a batch of unequal lengths, against the
plain implementation, in float32 and bfloat16.

  1b: Llama 3.2 1B (hidden 2048, 32 heads over 8 kv heads of 64, feed-forward 8192, vocabulary 128256, scaling factor 32)
  3b: Llama 3.2 3B layers (hidden 3072, 24 heads over 8 kv heads of 128: three query heads a group, feed-forward 8192)
  8b: Llama 3.1 8B layers (hidden 4096, 32 heads over 8 kv heads of 128, feed-forward 14336, untied head, factor 8)
The two larger ones have one layer and a vocabulary of 32003 to keep the plain implementation quick."""
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
SHAPES = {"1b": WIDE, "3b": WIDE_3B, "8b": WIDE_8B}


@pytest.fixture(scope="module", params=list(SHAPES))
def wide(request, tmp_path_factory):
    raw = SHAPES[request.param]
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
    # a prompt and then the last 8 tokens one by one
    (slot,) = eng.open(1)
    got = [eng.step([Entry(slot, seqs[0][:62], list(range(62)))]).cpu().numpy()]
    for t in seqs[0][62:]:
        got.append(eng.step([Entry(slot, [t], [0])]).cpu().numpy().copy())
    assert err(np.concatenate(got), want[0]) <= tol
    eng.close([slot])
