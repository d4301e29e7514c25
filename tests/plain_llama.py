"""A plain, slow implementation of the Llama dense decoder, for tests only.

Whole sequences, no cache, one function for each part, NumPy float64 unless a
dtype is given.  It is written from the formulas of computerex/dlgo (cited at
each function as path:line under the reference tree) and shares no code with
the package under test: it reads config.json and model.safetensors itself.

Where the reference has no text (llama3 frequency scaling, the pairing that
un-permuted projection rows need) the function says so and the tests pin it
by invariants instead.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ----------------------------------------------------------------------------
# reading a model folder (no code shared with the package)
# ----------------------------------------------------------------------------

def _bf16_to_f32(raw: np.ndarray) -> np.ndarray:
    """bfloat16 bits -> float32: a 16-bit left shift (quant/bf16.go:18-27)."""
    return (raw.astype(np.uint32) << 16).view(np.float32)


def read_safetensors(path: str) -> dict:
    """name -> float64 array.  Layout: u64 header length, JSON header, data."""
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
        data = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        buf = data[b:e]
        dt = info["dtype"]
        if dt == "BF16":
            arr = _bf16_to_f32(np.frombuffer(buf, dtype=np.uint16))
        elif dt == "F32":
            arr = np.frombuffer(buf, dtype=np.float32)
        elif dt == "F16":
            arr = np.frombuffer(buf, dtype=np.float16)
        else:
            raise ValueError(f"plain reader: dtype {dt} of {name}")
        out[name] = arr.astype(np.float64).reshape(info["shape"])
    return out


def read_model(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ----------------------------------------------------------------------------
# random weights from (seed, tensor name, element index), written a second time
# ----------------------------------------------------------------------------
# The recipe, as the library's documentation states it (the reference draws its fixtures from one seeded stream,
# testdata/generate.go:45-148; a counter keyed by name and index has no counterpart there):
#   key = splitmix64(seed ^ fnv1a64(name)); draw(c) = splitmix64(key + c * 0x9E3779B97F4A7C15), c = 1, 2, ...;
#   u(c) = ((draw(c) >> 11) + 1) / 2^53; normal i = sqrt(-2 ln u(2i+1)) cos(2 pi u(2i+2)); an element is
#   float32(offset + scale * normal i), then rounded to the stored type (bfloat16: nearest, ties to even).
# One element at a time with Python integers, so that nothing here resembles the vectorised code it checks.

_M64 = 0xFFFFFFFFFFFFFFFF


def _splitmix(z):
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def _fnv1a64(text):
    h = 0xCBF29CE484222325
    for byte in text.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _M64
    return h


def random_element(seed, name, i, scale, offset=0.0):
    """Element i (row-major) of tensor `name` for `seed`, as the float32 value before any narrower rounding."""
    key = _splitmix((seed & _M64) ^ _fnv1a64(name))
    u1 = ((_splitmix(key + (2 * i + 1) * 0x9E3779B97F4A7C15) >> 11) + 1) / 9007199254740992.0
    u2 = ((_splitmix(key + (2 * i + 2) * 0x9E3779B97F4A7C15) >> 11) + 1) / 9007199254740992.0
    normal = float(np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * math.pi * u2))
    return np.float32(offset + scale * normal) if offset else np.float32(scale * normal)


def round_to_bf16(x):
    """float32 -> the float32 value of the nearest bfloat16, ties to even (the rule of quant/bf16.go's inverse; NaNs do
    not occur here)."""
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)


def random_tensor(seed, name, shape, scale, offset=0.0, bf16=False):
    n = int(np.prod(shape))
    out = np.array([random_element(seed, name, i, scale, offset) for i in range(n)], dtype=np.float32)
    if bf16:
        out = round_to_bf16(out)
    return out.astype(np.float64).reshape(shape)


def llama_tensor_shapes(cfg):
    """name -> (shape, is a norm weight) for a Llama config.json, as a model folder names them."""
    d, f, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"]
    H = cfg["num_attention_heads"]
    KV = cfg.get("num_key_value_heads") or H
    hd = cfg.get("head_dim") or d // H
    out = {"model.embed_tokens.weight": ((cfg["vocab_size"], d), False), "model.norm.weight": ((d,), True)}
    if not cfg.get("tie_word_embeddings", False):
        out["lm_head.weight"] = ((cfg["vocab_size"], d), False)
    for l in range(L):
        p = f"model.layers.{l}."
        out[p + "input_layernorm.weight"] = ((d,), True)
        out[p + "post_attention_layernorm.weight"] = ((d,), True)
        out[p + "self_attn.q_proj.weight"] = ((H * hd, d), False)
        out[p + "self_attn.k_proj.weight"] = ((KV * hd, d), False)
        out[p + "self_attn.v_proj.weight"] = ((KV * hd, d), False)
        out[p + "self_attn.o_proj.weight"] = ((d, H * hd), False)
        out[p + "mlp.gate_proj.weight"] = ((f, d), False)
        out[p + "mlp.up_proj.weight"] = ((f, d), False)
        out[p + "mlp.down_proj.weight"] = ((d, f), False)
    return out


def random_model(cfg, seed, std=None, norm_jitter=0.0, bf16=False):
    """The weights of a Llama config.json for a seed, computed here: name -> float64 array."""
    std = cfg["initializer_range"] if std is None else std
    w = {}
    for name, (shape, is_norm) in llama_tensor_shapes(cfg).items():
        if is_norm:
            w[name] = random_tensor(seed, name, shape, norm_jitter, 1.0, bf16) if norm_jitter else np.ones(shape)
        else:
            w[name] = random_tensor(seed, name, shape, std, 0.0, bf16)
    return w


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def rmsnorm(x, w, eps):
    """out[i] = x[i] * (1/sqrt(sum(x^2)/n + eps)) * w[i]; no mean, no bias, the
    weight as it is (ops/norm.go:10-32, scale at :20)."""
    x = np.asarray(x)
    ss = np.sum(x * x, axis=-1, keepdims=True)
    scale = 1.0 / np.sqrt(ss / x.shape[-1] + eps)
    return x * scale * w


def rope_inv_freq(head_dim, theta, scaling=None):
    """theta_i = base^(-2i/hd) for pair i (ops/rope.go:16, models/llm/workers.go:165).

    The llama3 scaling of the frequencies is absent from the reference.  With
    wavelength lam = 2*pi/theta_i: shorter than P0/high keeps theta_i, longer
    than P0/low divides it by the factor, between them the two are blended
    linearly in (P0/lam - low)/(high - low).
    """
    half = head_dim // 2
    inv = np.array([1.0 / math.pow(float(theta), (2.0 * i) / head_dim) for i in range(half)])
    if scaling is None:
        return inv
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind == "default":
        return inv
    if kind != "llama3":
        raise ValueError(f"plain: rope_type {kind}")
    f = float(scaling["factor"])
    lo = float(scaling["low_freq_factor"])
    hi = float(scaling["high_freq_factor"])
    p0 = float(scaling["original_max_position_embeddings"])
    out = np.empty_like(inv)
    for i, th in enumerate(inv):
        lam = 2.0 * math.pi / th
        if lam < p0 / hi:
            out[i] = th
        elif lam > p0 / lo:
            out[i] = th / f
        else:
            s = (p0 / lam - lo) / (hi - lo)
            out[i] = (1.0 - s) * th / f + s * th
    return out


def rope_apply(v, pos, inv_freq, interleaved=False):
    """Rotate one head vector at absolute position pos (ops/rope.go:13-33).

    x0' = x0*cos - x1*sin ; x1' = x0*sin + x1*cos with angle pos*theta_i.
    split-half pairs (v[i], v[i+hd/2]) (rope.go:21-25), interleaved pairs
    (v[2i], v[2i+1]) (rope.go:26-31).  Projection rows named as in a
    config.json/safetensors folder are not permuted, so they take split-half.
    """
    v = np.asarray(v, dtype=np.float64)
    half = v.shape[-1] // 2
    ang = pos * inv_freq
    c, s = np.cos(ang), np.sin(ang)
    out = np.empty_like(v)
    if interleaved:
        x0, x1 = v[..., 0::2], v[..., 1::2]
        out[..., 0::2] = x0 * c - x1 * s
        out[..., 1::2] = x0 * s + x1 * c
    else:
        x0, x1 = v[..., :half], v[..., half:]
        out[..., :half] = x0 * c - x1 * s
        out[..., half:] = x0 * s + x1 * c
    return out


def softmax(x):
    """max-subtracted softmax (ops/ops.go:150-170), with an exact exp."""
    x = np.asarray(x, dtype=np.float64)
    e = np.exp(x - np.max(x))
    return e / np.sum(e)


def attention(q, k, v, n_heads, n_kv_heads, head_dim, window=None):
    """Causal grouped-query attention over one whole sequence.

    q [T, H*hd], k, v [T, KV*hd], already rotated.  Query head h reads KV head
    h // (H/KV); token p sees keys 0..p, the mask being the loop bound
    seqLen = p+1; scale 1/sqrt(hd) (models/llm/forward.go:258-278,
    layers/gqa.go:22-48).  With a window, token p sees keys
    max(0, p-window+1)..p (layers/gqa.go:98-132).
    """
    T = q.shape[0]
    g = n_heads // n_kv_heads
    scale = 1.0 / math.sqrt(head_dim)
    out = np.zeros((T, n_heads * head_dim))
    for h in range(n_heads):
        kvh = h // g
        qs = slice(h * head_dim, (h + 1) * head_dim)
        ks = slice(kvh * head_dim, (kvh + 1) * head_dim)
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            scores = (k[lo:p + 1, ks] @ q[p, qs]) * scale        # one dot product per visible key
            pr = softmax(scores)
            out[p, qs] = pr @ v[lo:p + 1, ks]                    # the values, weighted
    return out


def silu(z):
    """z / (1 + exp(-z)) (ops/activation.go:36-38)."""
    return z / (1.0 + np.exp(-z))


def swiglu(gate, up):
    """silu(gate) * up (ops/activation.go:8-19)."""
    return silu(np.asarray(gate, dtype=np.float64)) * up


def feed_forward(x, w_gate, w_up, w_down):
    """down( silu(gate x) * (up x) ), no biases (models/llm/forward.go:295-298)."""
    return swiglu(x @ w_gate.T, x @ w_up.T) @ w_down.T


def block(x, positions, w, prefix, cfg, inv_freq, window=None):
    """x -> x + O(attn(rope(Q,K),V)) ; -> + FFN(norm) (models/llm/forward.go:137-169)."""
    H = cfg["num_attention_heads"]
    KV = cfg.get("num_key_value_heads", H)
    hd = cfg.get("head_dim", cfg["hidden_size"] // H)
    eps = cfg["rms_norm_eps"]
    xn = rmsnorm(x, w[prefix + "input_layernorm.weight"], eps)
    q = xn @ w[prefix + "self_attn.q_proj.weight"].T
    k = xn @ w[prefix + "self_attn.k_proj.weight"].T
    v = xn @ w[prefix + "self_attn.v_proj.weight"].T
    if prefix + "self_attn.q_proj.bias" in w:          # biases where the layer has them (models/llm/forward.go:227-235)
        q = q + w[prefix + "self_attn.q_proj.bias"]
        k = k + w[prefix + "self_attn.k_proj.bias"]
        v = v + w[prefix + "self_attn.v_proj.bias"]
    T = x.shape[0]
    for t in range(T):
        q[t] = rope_apply(q[t].reshape(H, hd), positions[t], inv_freq).reshape(-1)
        k[t] = rope_apply(k[t].reshape(KV, hd), positions[t], inv_freq).reshape(-1)
    a = attention(q, k, v, H, KV, hd, window)
    h = x + a @ w[prefix + "self_attn.o_proj.weight"].T
    if prefix + "self_attn.o_proj.bias" in w:          # (models/llm/forward.go:286-289)
        h = h + w[prefix + "self_attn.o_proj.bias"]
    hn = rmsnorm(h, w[prefix + "post_attention_layernorm.weight"], eps)
    f = feed_forward(hn, w[prefix + "mlp.gate_proj.weight"], w[prefix + "mlp.up_proj.weight"],
                     w[prefix + "mlp.down_proj.weight"])
    return h + f


def forward(cfg, w, tokens, start_pos=0, rows=None):
    """Logits [T, V] of one whole sequence (models/llm/forward.go:123-204):
    embedding row, L blocks, final norm, output matrix (the embedding table
    when tied, models/llm/loader.go:74-76).  rows: the positions whose logits
    are wanted (all of them if None); the blocks always see the whole sequence."""
    H = cfg["num_attention_heads"]
    hd = cfg.get("head_dim", cfg["hidden_size"] // H)
    inv_freq = rope_inv_freq(hd, cfg["rope_theta"], cfg.get("rope_scaling"))
    tokens = list(tokens)
    for t in tokens:
        if not 0 <= t < cfg["vocab_size"]:
            raise ValueError(f"token {t} out of range")
    x = w["model.embed_tokens.weight"][tokens].astype(np.float64)
    positions = [start_pos + i for i in range(len(tokens))]
    for l in range(cfg["num_hidden_layers"]):
        x = block(x, positions, w, f"model.layers.{l}.", cfg, inv_freq)
    if rows is not None:
        x = x[list(rows)]
    x = rmsnorm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    out_w = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ out_w.T


# ----------------------------------------------------------------------------
# sampling (ops/sampling.go)
# ----------------------------------------------------------------------------

def argmax(x):
    """First maximum; -1 when empty (ops/ops.go:272-285)."""
    if len(x) == 0:
        return -1
    best, idx = x[0], 0
    for i in range(1, len(x)):
        if x[i] > best:
            best, idx = x[i], i
    return idx


def apply_repetition_penalty(logits, recent, penalty):
    """Each distinct recent token once: positive logits divided, others
    multiplied (ops/sampling.go:53-69)."""
    out = np.array(logits, dtype=np.float64)
    if penalty <= 1.0 or len(recent) == 0:
        return out
    for tok in set(int(t) for t in recent):
        if 0 <= tok < len(out):
            out[tok] = out[tok] / penalty if out[tok] > 0 else out[tok] * penalty
    return out


def apply_temperature(logits, temp):
    """logits * (1/temp), skipped for temp <= 0 or 1 (ops/sampling.go:72-80)."""
    out = np.array(logits, dtype=np.float64)
    if temp <= 0 or temp == 1.0:
        return out
    return out * (1.0 / temp)


def apply_top_k(logits, k):
    """Below the k-th largest value -> -inf; ties at it stay (ops/sampling.go:83-95)."""
    out = np.array(logits, dtype=np.float64)
    if k <= 0 or k >= len(out):
        return out
    cutoff = np.sort(out)[::-1][k - 1]
    out[out < cutoff] = -np.inf
    return out


def apply_top_p(logits, p):
    """Smallest set, by falling probability, whose mass reaches p
    (ops/sampling.go:99-138).  Equal probabilities at the cut are all kept
    here; the reference's unstable sort keeps an unspecified subset of them."""
    out = np.array(logits, dtype=np.float64)
    if p >= 1.0:
        return out
    probs = softmax(out)
    order = np.argsort(-probs, kind="stable")
    cum = np.cumsum(probs[order])
    cut = int(np.searchsorted(cum, p, side="left"))
    cut = min(cut, len(out) - 1)
    thresh = probs[order[cut]]
    out[probs < thresh] = -np.inf
    return out


def apply_min_p(logits, min_p):
    """Probability below min_p * max probability -> -inf (ops/sampling.go:143-165)."""
    out = np.array(logits, dtype=np.float64)
    if min_p <= 0:
        return out
    probs = softmax(out)
    out[probs < min_p * probs.max()] = -np.inf
    return out


def sample_from_logits(logits, r):
    """softmax, then the first i whose running sum reaches r, else the last
    index (ops/sampling.go:167-181)."""
    probs = softmax(logits)
    cum = 0.0
    for i, p in enumerate(probs):
        cum += p
        if cum >= r:
            return i
    return len(probs) - 1


def filtered_logits(logits, temperature, top_k=0, top_p=1.0, min_p=0.0, penalty=1.0, recent=()):
    """What the draw is taken from: penalty -> temperature -> top-k -> top-p -> min-p (ops/sampling.go:36-47)."""
    w = apply_repetition_penalty(logits, recent, penalty)
    w = apply_temperature(w, temperature)
    w = apply_top_k(w, top_k)
    w = apply_top_p(w, top_p)
    return apply_min_p(w, min_p)


def sample_token(logits, r, temperature, top_k=0, top_p=1.0, min_p=0.0, penalty=1.0, recent=()):
    """penalty -> temperature -> top-k -> top-p -> min-p -> draw; temperature
    <= 0 is greedy (ops/sampling.go:32-48)."""
    if temperature <= 0:
        return argmax(logits)
    return sample_from_logits(filtered_logits(logits, temperature, top_k, top_p, min_p, penalty, recent), r)


def greedy_generate(cfg, w, prompt, max_tokens, stop_tokens=()):
    """Public-path loop (models/llm/generate.go:340-386): sample, a stop token
    ends the run and is not emitted, else append and feed it back."""
    seq = list(prompt)
    out = []
    for _ in range(max_tokens):
        nxt = argmax(forward(cfg, w, seq)[-1])
        if nxt in stop_tokens:
            break
        out.append(nxt)
        seq.append(nxt)
    return out
