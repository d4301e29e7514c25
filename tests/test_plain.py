"""What fixes the plain implementation beside the reference's text: the reference's own test
vectors, special cases that reduce to a library routine, and invariants, each chosen so that a
plausible mistake fails it."""
import math

import numpy as np
import pytest

import plain_llama as plain
from conftest import TINY_A, TINY_B, llama3_blend_cases


# -- RMSNorm -------------------------------------------------------------------
def test_rmsnorm_reference_vectors():
    # ops/norm_test.go:8-22
    out = plain.rmsnorm(np.array([1., 2., 3., 4.]), np.ones(4), 1e-5)
    assert np.allclose(out, np.array([1., 2., 3., 4.]) / math.sqrt(7.5 + 1e-5), atol=1e-12)
    # ops/norm_test.go:24-38
    out = plain.rmsnorm(np.array([2., 4., 6.]), np.full(3, 0.5), 1e-5)
    assert np.allclose(out, 0.5 * np.array([2., 4., 6.]) / math.sqrt(56 / 3 + 1e-5), atol=1e-12)
    # ops/norm_test.go:40-52: equal inputs -> the weights themselves (a weight applied as 1+w fails this)
    out = plain.rmsnorm(np.ones(4), np.array([2., 3., 4., 5.]), 1e-5)
    assert np.allclose(out, np.array([2., 3., 4., 5.]), atol=1e-4)


def test_rmsnorm_invariants():
    rng = np.random.default_rng(0)
    x, w = rng.normal(size=16), rng.normal(size=16)
    # scale invariance as eps -> 0, and no mean subtraction (a constant shift changes the result)
    assert np.allclose(plain.rmsnorm(7.0 * x, w, 1e-30), plain.rmsnorm(x, w, 1e-30))
    assert not np.allclose(plain.rmsnorm(x + 5.0, w, 1e-30), plain.rmsnorm(x, w, 1e-30))
    # eps sits inside the root, added to the mean square
    tiny = 1e-4 * x
    want = tiny / np.sqrt((tiny * tiny).mean() + 1e-5) * w
    assert np.allclose(plain.rmsnorm(tiny, w, 1e-5), want)
    assert not np.allclose(plain.rmsnorm(tiny, w, 1e-5), plain.rmsnorm(tiny, w, 1e-6))


# -- RoPE ----------------------------------------------------------------------
def test_rope_reference_vectors():
    inv = plain.rope_inv_freq(8, 10000.0)
    v = np.arange(1., 9.)
    for inter in (False, True):                                  # ops/rope_test.go:8-34,107-129
        assert np.array_equal(plain.rope_apply(v, 0, inv, inter), v)
    out = plain.rope_apply(np.array([1., 0.]), 1, plain.rope_inv_freq(2, 1.0), True)   # ops/rope_test.go:36-47
    assert np.allclose(out, [math.cos(1), math.sin(1)])
    # theta_i = base^(-2i/hd)
    assert np.allclose(plain.rope_inv_freq(8, 10000.0), [1, 10000 ** -0.25, 10000 ** -0.5, 10000 ** -0.75])


def test_rope_invariants():
    rng = np.random.default_rng(1)
    hd = 16
    inv = plain.rope_inv_freq(hd, 500000.0)
    q, k = rng.normal(size=hd), rng.normal(size=hd)
    for inter in (False, True):
        # norms of pairs survive; scores depend on the distance only (a wrong sign breaks this)
        assert np.isclose(np.linalg.norm(plain.rope_apply(q, 37, inv, inter)), np.linalg.norm(q))
        a = plain.rope_apply(q, 40, inv, inter) @ plain.rope_apply(k, 33, inv, inter)
        b = plain.rope_apply(q, 107, inv, inter) @ plain.rope_apply(k, 100, inv, inter)
        c = plain.rope_apply(q, 33, inv, inter) @ plain.rope_apply(k, 40, inv, inter)
        assert np.isclose(a, b) and not np.isclose(a, c)
    # split-half is interleaved under the fixed permutation [0,2,4,...,1,3,5,...]
    perm = np.concatenate([np.arange(0, hd, 2), np.arange(1, hd, 2)])
    assert np.allclose(plain.rope_apply(q, 9, inv, True)[perm], plain.rope_apply(q[perm], 9, inv, False))
    # split-half pairs element i with i + hd/2: rotating a vector with only element 0 set moves weight to hd/2
    e0 = np.zeros(hd)
    e0[0] = 1
    out = plain.rope_apply(e0, 1, inv, False)
    assert np.isclose(out[0], math.cos(1)) and np.isclose(out[hd // 2], math.sin(1)) and np.isclose(abs(out).sum(), abs(math.cos(1)) + abs(math.sin(1)))


def test_llama3_scaling_invariants():
    base = plain.rope_inv_freq(32, 500000.0)
    sc = dict(TINY_B["rope_scaling"])
    scaled = plain.rope_inv_freq(32, 500000.0, sc)
    assert np.array_equal(plain.rope_inv_freq(32, 500000.0, None), base)
    assert np.allclose(plain.rope_inv_freq(32, 500000.0, dict(sc, factor=1.0)), base)
    assert np.all(np.diff(scaled) <= 0)
    # regimes of this configuration: pairs 0-1 kept bit for bit, pair 2 blended, pairs 3.. divided by 4
    assert np.array_equal(scaled[:2], base[:2])
    assert base[2] / 4 < scaled[2] < base[2]
    assert np.allclose(scaled[3:], base[3:] / 4)
    # the 1B shape: 0-14 kept, 15-17 blended, 18-31 divided by 32
    big = dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
    b64, s64 = plain.rope_inv_freq(64, 500000.0), plain.rope_inv_freq(64, 500000.0, big)
    assert np.array_equal(s64[:15], b64[:15]) and np.allclose(s64[18:], b64[18:] / 32)
    assert all(b64[i] / 32 < s64[i] < b64[i] for i in (15, 16, 17))


def test_llama3_blend_on_constructed_wavelengths():
    """The blend itself, through the implementation: s = 1/2, 1/4, 3/4 exactly and both edges.  A blend with s and 1-s
    exchanged fails the quarter points and the edges, a constant half fails them too, and a geometric blend
    (theta * f^-(1-s)) fails the midpoint."""
    for theta, sc, want, tol in llama3_blend_cases():
        got = plain.rope_inv_freq(4, theta, sc)
        assert got[0] == 1.0                                  # wavelength 2 pi: far below P0/high, kept bit for bit
        assert math.isclose(got[1], want, rel_tol=tol), (theta, got[1], want)

# -- attention -----------------------------------------------------------------
def test_attention_reference_vectors():
    rng = np.random.default_rng(2)
    H, KV, hd = 4, 2, 8
    # one position: output = V for every head of the group (layers/gqa_test.go:8-43)
    q, k, v = rng.normal(size=(1, H * hd)), rng.normal(size=(1, KV * hd)), rng.normal(size=(1, KV * hd))
    out = plain.attention(q, k, v, H, KV, hd)
    assert np.allclose(out.reshape(H, hd), np.repeat(v.reshape(KV, hd), 2, axis=0))
    # equal keys: the plain mean; with window 2 at position 3 of v=0,1,2,3 -> 2.5 (layers/gqa_test.go:110-136)
    k = np.ones((4, hd))
    v = np.repeat(np.arange(4.)[:, None], hd, axis=1)
    q = rng.normal(size=(4, hd))
    assert np.allclose(plain.attention(q, k, v, 1, 1, hd, window=2)[3], 2.5)
    assert np.allclose(plain.attention(q, k, v, 1, 1, hd)[3], 1.5)
    assert np.allclose(plain.attention(q, k, v, 1, 1, hd)[0], 0.0)          # causal: position 0 sees V[0] only


def test_attention_is_library_softmax_attention():
    """Without rotation: softmax(QK^T/sqrt(hd) + causal mask) V with K/V heads repeated, in float64."""
    rng = np.random.default_rng(3)
    T, H, KV, hd = 9, 6, 2, 8
    q, k, v = rng.normal(size=(T, H * hd)), rng.normal(size=(T, KV * hd)), rng.normal(size=(T, KV * hd))
    got = plain.attention(q, k, v, H, KV, hd)
    qh = q.reshape(T, H, hd).transpose(1, 0, 2)
    kh = np.repeat(k.reshape(T, KV, hd).transpose(1, 0, 2), H // KV, axis=0)
    vh = np.repeat(v.reshape(T, KV, hd).transpose(1, 0, 2), H // KV, axis=0)
    s = qh @ kh.transpose(0, 2, 1) / math.sqrt(hd)
    s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = (p @ vh).transpose(1, 0, 2).reshape(T, H * hd)
    assert np.allclose(got, want)
    # a token ignores later rows: poisoning them changes nothing before
    k2, v2 = k.copy(), v.copy()
    k2[5:], v2[5:] = np.nan, np.nan
    assert np.allclose(plain.attention(q, k2, v2, H, KV, hd)[:5], want[:5])
    # one kv head per query head is plain multi-head attention (layers/gqa_test.go:45-72)
    kk, vv = rng.normal(size=(T, H * hd)), rng.normal(size=(T, H * hd))
    one = plain.attention(q, kk, vv, H, H, hd)
    for h in range(H):
        sl = slice(h * hd, (h + 1) * hd)
        assert np.allclose(one[:, sl], plain.attention(q[:, sl], kk[:, sl], vv[:, sl], 1, 1, hd))


def test_softmax():
    p = plain.softmax(np.array([1., 2., 3.]))
    assert np.isclose(p.sum(), 1) and np.allclose(p, plain.softmax(np.array([101., 102., 103.])))   # ops/ops_test.go:121-134


# -- feed-forward ----------------------------------------------------------------
def test_swiglu_reference_vectors():
    g = np.array([0., 1., -1., 2.])
    assert np.allclose(plain.swiglu(g, np.ones(4)), g / (1 + np.exp(-g)))      # ops/activation_test.go:16-28
    assert np.array_equal(plain.swiglu(np.zeros(3), np.array([5., -2., 9.])), np.zeros(3))   # :44-53
    assert np.isclose(plain.swiglu(np.array([1.]), np.array([2.]))[0], 1.4621, atol=1e-4)    # quant/quant_extended_test.go:312-326
    # gate and up are not interchangeable
    assert not np.isclose(plain.swiglu(np.array([2.]), np.array([1.]))[0], plain.swiglu(np.array([1.]), np.array([2.]))[0])


# -- sampling ----------------------------------------------------------------------
def test_sampling_reference_vectors():
    assert plain.argmax(np.array([1., 5., 2., 3.])) == 1                      # ops/sampling_test.go:9-16
    assert plain.argmax(np.array([])) == -1 and plain.argmax(np.array([2., 7., 7.])) == 1    # ops/ops_test.go:175-183
    assert np.allclose(plain.apply_temperature([2., 4., 6.], 2.0), [1., 2., 3.])             # sampling_test.go:48-57
    out = plain.apply_top_k([1., 4., 2., 5., 3.], 2)                                         # :59-70
    assert np.isinf(out[[0, 2, 4]]).all() and list(out[[1, 3]]) == [4., 5.]
    assert np.allclose(plain.apply_repetition_penalty([2., -1., 3., 0.], [0, 1], 2.0), [1., -2., 3., 0.])   # :32-46
    big = np.zeros(10)
    big[4] = 100.0
    assert all(plain.sample_token(big, r, 1.0) == 4 for r in np.linspace(0.001, 0.999, 100))     # :18-30
    # top-p keeps the smallest set that reaches p
    lg = np.log(np.array([0.5, 0.3, 0.15, 0.05]))
    assert np.isinf(plain.apply_top_p(lg, 0.7)).tolist() == [False, False, True, True]
    assert np.isinf(plain.apply_min_p(lg, 0.5)).tolist() == [False, False, True, True]
    # the draw: first index whose running sum reaches r
    assert [plain.sample_from_logits(lg, r) for r in (0.1, 0.5, 0.51, 0.81, 0.96)] == [0, 0, 1, 2, 3]


# -- whole model -----------------------------------------------------------------
def _tiny(raw, seed, tmp_path, **kw):
    from conftest import make_folder
    return plain.read_model(make_folder(raw, seed, tmp_path, **kw))


def test_forward_sanity_and_position_shift(tmp_path):
    cfg, w = _tiny(TINY_A, 3, tmp_path, std=0.1)
    toks = [5, 17, 3, 200, 41, 7]
    a = plain.forward(cfg, w, toks)
    assert a.shape == (6, 256) and np.isfinite(a).all() and a.std() > 1e-3
    # rotary attention sees distances only: shifting every position changes nothing (no scaling in this config)
    assert np.allclose(a, plain.forward(cfg, w, toks, start_pos=50), atol=1e-9)
    # causal: a prefix's logits do not depend on what follows; and the context matters
    assert np.allclose(a[:3], plain.forward(cfg, w, toks[:3]))
    assert not np.allclose(a[-1], plain.forward(cfg, w, [9] + toks[1:])[-1])
    with pytest.raises(ValueError):
        plain.forward(cfg, w, [256])


def test_tied_and_untied_heads(tmp_path):
    cfg, w = _tiny(TINY_A, 4, tmp_path / "a")
    assert "lm_head.weight" not in w
    cfg_b, w_b = _tiny(TINY_B, 5, tmp_path / "b", norm_jitter=0.1)
    toks = [1, 2, 3]
    base = plain.forward(cfg_b, w_b, toks)
    w2 = dict(w_b)
    w2["lm_head.weight"] = w_b["lm_head.weight"] * 2.0
    assert np.allclose(plain.forward(cfg_b, w2, toks), 2.0 * base)        # the head is last and linear
    w3 = dict(w_b)
    w3["model.embed_tokens.weight"] = w_b["model.embed_tokens.weight"] * 1.5
    assert not np.allclose(plain.forward(cfg_b, w3, toks), base)


def test_greedy_generate_stops(tmp_path):
    cfg, w = _tiny(TINY_A, 6, tmp_path, std=0.1)
    out = plain.greedy_generate(cfg, w, [1, 2, 3], 5)
    assert len(out) == 5
    # the stop token is not emitted (decode/decode_test.go:8-30); an immediate one gives nothing (:39-51)
    assert plain.greedy_generate(cfg, w, [1, 2, 3], 5, stop_tokens=(out[2],)) == out[:out.index(out[2])]
    assert plain.greedy_generate(cfg, w, [1, 2, 3], 5, stop_tokens=(out[0],)) == []
