"""LlamaConfig: the keys of a Llama config.json, typed and checked.

Stands where computerex/dlgo's parseConfig stands (models/llm/config.go:43-123):
`hidden_size` for `.embedding_length` (:70), `num_hidden_layers` for
`.block_count` (:71), `intermediate_size` for `.feed_forward_length` (:72),
`num_attention_heads` / `num_key_value_heads` for `.attention.head_count[_kv]`
(:73-74, kv defaulting to the head count :100-102), `head_dim` for
`.attention.key_length` (defaulting to hidden/heads, :103-105), `rms_norm_eps`
for `.attention.layer_norm_rms_epsilon` (:61-64), `rope_theta` for
`.rope.freq_base` (:77), `max_position_embeddings` for `.context_length` (:69),
eos/bos ids (:78-79,114-120).  dlgo falls back to constants where a key is
absent; here the numbers a model's arithmetic depends on must be in the file.
The llama3 `rope_scaling` block has no counterpart in dlgo.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class RopeScaling:
    """The llama3 recipe for stretching low rotary frequencies."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    def to_dict(self) -> Dict[str, Any]:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


def _read_rope_scaling(r: KeyReader) -> Optional[RopeScaling]:
    raw = r.raw.get("rope_scaling")
    if raw is None:
        return None
    if not isinstance(raw, Mapping):
        r.complain(f"rope_scaling: expected an object or null, found {raw!r}")
        return None
    kind = raw.get("rope_type", raw.get("type"))
    if kind == "default":
        return None
    if kind != "llama3":
        r.complain(f"rope_scaling.rope_type: only \"llama3\" (or \"default\"/null) is supported, found {kind!r}")
        return None
    sub = KeyReader(raw, "rope_scaling")
    factor = sub.number("factor", positive=True)
    lo = sub.number("low_freq_factor", positive=True)
    hi = sub.number("high_freq_factor", positive=True)
    p0 = sub.integer("original_max_position_embeddings", minimum=1)
    for p in sub.problems:
        r.complain("rope_scaling." + p)
    if sub.problems:
        return None
    if not hi > lo:
        r.complain(f"rope_scaling: high_freq_factor ({hi}) must exceed low_freq_factor ({lo})")
        return None
    return RopeScaling("llama3", factor, lo, hi, p0)


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    max_position_embeddings: int
    tie_word_embeddings: bool
    attention_bias: bool
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    initializer_range: Optional[float]
    torch_dtype: str

    # sizes derived once (dlgo recomputes them at each use, models/llm/forward.go:53-55)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    # what the rest of the library asks of any configuration
    def context_length(self) -> Optional[int]:
        return self.max_position_embeddings

    def stop_tokens(self) -> Tuple[int, ...]:
        return self.eos_token_ids

    def describe(self) -> List[str]:
        return [f"{self.num_hidden_layers} layers", f"{self.hidden_size} dim",
                f"{self.num_attention_heads} heads ({self.num_key_value_heads} KV)", f"{self.intermediate_size} FFN",
                f"vocab {self.vocab_size}"]

    def storage_dtype(self) -> str:
        return self.torch_dtype

    def init_std(self) -> Optional[float]:
        return self.initializer_range

    def stored_as(self, dtype_name: str) -> "LlamaConfig":
        return replace(self, torch_dtype=dtype_name)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "LlamaConfig":
        r = KeyReader(raw)
        names = raw.get("architectures")
        arch = names[0] if isinstance(names, (list, tuple)) and names else names
        vocab = r.integer("vocab_size", minimum=1)
        d = r.integer("hidden_size", minimum=1)
        layers = r.integer("num_hidden_layers", minimum=1)
        ffn = r.integer("intermediate_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv = r.integer("num_key_value_heads", default=heads, minimum=1)
        hd_default = (d // heads) if (d and heads) else _no_default()
        hd = r.integer("head_dim", default=hd_default, minimum=1)
        eps = r.number("rms_norm_eps", positive=True)
        theta = r.number("rope_theta", positive=True)
        scaling = _read_rope_scaling(r)
        max_pos = r.integer("max_position_embeddings", minimum=1)
        tie = r.boolean("tie_word_embeddings", default=False)
        bos = r.integer("bos_token_id", default=None, minimum=0)
        init_range = r.number("initializer_range", default=None, positive=True)
        dtype = r.string("torch_dtype", default=raw.get("dtype") or "bfloat16")

        eos_raw = raw.get("eos_token_id")
        eos: Tuple[int, ...] = ()
        if eos_raw is not None:
            items = eos_raw if isinstance(eos_raw, (list, tuple)) else [eos_raw]
            if all(isinstance(t, int) and not isinstance(t, bool) and t >= 0 for t in items):
                eos = tuple(items)
            else:
                r.complain(f"eos_token_id: expected a token id or a list of them, found {eos_raw!r}")

        attention_bias = r.boolean("attention_bias", default=False)
        if r.boolean("mlp_bias", default=False):
            r.complain("mlp_bias: feed-forward biases have no kernel here (the gate/up product ends in SwiGLU directly)")
        act = r.string("hidden_act", default="silu")
        if act is not None and act != "silu":
            r.complain(f"hidden_act: only \"silu\" (SwiGLU) is supported, found {act!r}")
        if dtype is not None and dtype not in ("bfloat16", "float32", "float16"):
            r.complain(f"torch_dtype: expected bfloat16, float16 or float32, found {dtype!r}")

        if heads and kv and heads % kv != 0:
            r.complain(f"num_attention_heads ({heads}) must be a multiple of num_key_value_heads ({kv})")
        if hd and hd % 2 != 0:
            r.complain(f"head_dim ({hd}) must be even for rotary pairs")
        if vocab:
            for name, tok in (("bos_token_id", bos),) + tuple(("eos_token_id", t) for t in eos):
                if tok is not None and tok >= vocab:
                    r.complain(f"{name} ({tok}) is outside the vocabulary ({vocab})")
        r.finish()
        return cls(architecture=arch, vocab_size=vocab, hidden_size=d, num_hidden_layers=layers,
                   intermediate_size=ffn, num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd,
                   rms_norm_eps=eps, rope_theta=theta, rope_scaling=scaling, max_position_embeddings=max_pos,
                   tie_word_embeddings=tie, attention_bias=bool(attention_bias), bos_token_id=bos, eos_token_ids=eos,
                   initializer_range=init_range, torch_dtype=dtype)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "intermediate_size": self.intermediate_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.initializer_range is not None:
            out["initializer_range"] = self.initializer_range
        return out


def _no_default():
    from .base import _MISSING
    return _MISSING
