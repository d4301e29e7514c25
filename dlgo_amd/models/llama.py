"""The Llama dense decoder, put together from parts according to a LlamaConfig.

Every layer has the same description here, but the description is per layer:
computerex/dlgo resolves a LayerSpec for each layer (models/llm/loader.go:88-125),
which for this architecture is {RMSNorm, attention, standard residual, SwiGLU}
(models/llm/model.go:12-55).  Tensor names are those of a config.json/safetensors
folder: model.embed_tokens, model.layers.{i}.{input_layernorm, self_attn.{q,k,v,o}_proj,
post_attention_layernorm, mlp.{gate,up,down}_proj}, model.norm, lm_head; with
`attention_bias` the four attention projections also have a `.bias` each (the reference adds
biases where a layer has them, models/llm/forward.go:227-235).
Projection rows in such a folder are not permuted, so the rotary pairing is
split-half (the reference's interleaved pairing for "llama", models/llm/arch.go:18,
suits the permuted rows of its own file format).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

from ..config import LlamaConfig, register_architecture
from ..parts import DecoderModel, Embedding, LayerRun, OutputHead, make_part


@dataclass(frozen=True)
class LayerSpec:
    """The independent choices of one layer, by registered name."""
    block: str = "pre_norm"
    norm: str = "rmsnorm"
    mixer: str = "attention"
    feed_forward: str = "gated"
    position: str = "rotary"
    window: Optional[int] = None


def layer_specs(config: LlamaConfig) -> List[LayerSpec]:
    return [LayerSpec() for _ in range(config.num_hidden_layers)]


def build_llama(config: LlamaConfig) -> DecoderModel:
    d = config.hidden_size
    layers = []
    for i, spec in enumerate(layer_specs(config)):
        position = make_part("position", spec.position, config.head_dim, config.rope_theta, config.rope_scaling)
        mixer = make_part("mixer", spec.mixer, d, config.num_attention_heads, config.num_key_value_heads, config.head_dim,
                          position, window=spec.window, bias=config.attention_bias, out_bias=config.attention_bias)
        ffn = make_part("feed_forward", spec.feed_forward, d, config.intermediate_size, "silu")
        block = make_part("block", spec.block,
                          ("input_layernorm", make_part("norm", spec.norm, d, config.rms_norm_eps)),
                          ("self_attn", mixer),
                          ("post_attention_layernorm", make_part("norm", spec.norm, d, config.rms_norm_eps)),
                          ("mlp", ffn))
        layers.append((f"model.layers.{i}", block))
    embedding = Embedding(config.vocab_size, d)
    head = OutputHead(config.vocab_size, d, tied_to=embedding if config.tie_word_embeddings else None)
    return DecoderModel(
        config,
        embedding=("model.embed_tokens", embedding),
        layers=layers,
        final_norm=("model.norm", make_part("norm", "rmsnorm", d, config.rms_norm_eps)),
        head=("lm_head", head),
        order=[LayerRun(i) for i in range(config.num_hidden_layers)],
        # a tied model's file may still carry the head's copy of the table
        ignorable_tensors=("lm_head.weight",) if config.tie_word_embeddings else (),
    )


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama)
