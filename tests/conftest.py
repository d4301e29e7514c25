import copy
import math
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 256, "hidden_size": 64, "num_hidden_layers": 2, "intermediate_size": 160,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "max_position_embeddings": 128, "tie_word_embeddings": True, "initializer_range": 0.02,
    "hidden_act": "silu", "torch_dtype": "float32", "bos_token_id": 1, "eos_token_id": 2,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 384, "hidden_size": 128, "num_hidden_layers": 3, "intermediate_size": 352,
    "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 32,
    "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "max_position_embeddings": 512, "tie_word_embeddings": False, "initializer_range": 0.02,
    "hidden_act": "silu", "torch_dtype": "float32", "bos_token_id": 0, "eos_token_id": [3, 5],
}
# a third one with a head size that is neither a power of two nor hidden/heads, and more heads than fit one wave's tile
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 515, "hidden_size": 96, "num_hidden_layers": 2, "intermediate_size": 136,
    "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48,
    "rms_norm_eps": 3e-6, "rope_theta": 20000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 2.0,
                     "original_max_position_embeddings": 32},
    "max_position_embeddings": 640, "tie_word_embeddings": True, "initializer_range": 0.05,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": 7,
}


@pytest.fixture
def tiny_a():
    return copy.deepcopy(TINY_A)


@pytest.fixture
def tiny_b():
    return copy.deepcopy(TINY_B)
# a fourth one: a head size of 80 (above 64, no power of two), one kv head for eight query heads, no scaling of the rotation
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 1000, "hidden_size": 200, "num_hidden_layers": 2, "intermediate_size": 264,
    "num_attention_heads": 8, "num_key_value_heads": 1, "head_dim": 80,
    "rms_norm_eps": 1e-4, "rope_theta": 1000000.0, "rope_scaling": None,
    "max_position_embeddings": 1024, "tie_word_embeddings": False, "initializer_range": 0.04,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "eos_token_id": [3, 4],
}


@pytest.fixture
def tiny_c():
    return copy.deepcopy(TINY_C)


def make_folder(raw, seed, path, dtype=None, std=None, norm_jitter=0.0):
    """Write a random model folder for a raw config dict with the library's own writer."""
    import torch
    from dlgo_amd import models  # noqa: F401
    from dlgo_amd.config import config_from_dict
    from dlgo_amd.weights import write_random_model
    dt = {None: None, "float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    return write_random_model(config_from_dict(raw), seed, str(path), dtype=dt, std=std, norm_jitter=norm_jitter)


def llama3_blend_cases():
    """Constructed configurations whose second pair of a head of size 4 has a chosen wavelength, with the frequency the
    llama3 recipe must give it: (theta, scaling dict, wanted frequency of pair 1, tolerance).  P0 = 64, low 1, high 4:
    wavelengths between 16 and 64 are blended with s = (P0/wavelength - low)/(high - low).  Pair 1 of a head of size 4
    has frequency base^(-1/2), so base = (wavelength / 2 pi)^2 places it."""
    p0, lo, hi, f = 64.0, 1.0, 4.0, 8.0
    sc = dict(rope_type="llama3", factor=f, low_freq_factor=lo, high_freq_factor=hi, original_max_position_embeddings=int(p0))
    cases = []
    for ratio, weight_of_unscaled in ((2.5, 0.5), (1.75, 0.25), (3.25, 0.75)):      # P0/wavelength -> s
        lam = p0 / ratio
        th = 2.0 * math.pi / lam
        cases.append(((lam / (2.0 * math.pi)) ** 2, sc, th * ((1.0 - weight_of_unscaled) / f + weight_of_unscaled), 1e-12))
    # just inside either edge of the blend: close to the regime next to it
    for lam, factor in ((p0 / hi * (1 + 1e-7), 1.0), (p0 / lo * (1 - 1e-7), 1.0 / f)):
        cases.append(((lam / (2.0 * math.pi)) ** 2, sc, 2.0 * math.pi / lam * factor, 1e-5))
    # just outside: exactly the regime
    for lam, factor in ((p0 / hi * (1 - 1e-7), 1.0), (p0 / lo * (1 + 1e-7), 1.0 / f)):
        cases.append(((lam / (2.0 * math.pi)) ** 2, sc, 2.0 * math.pi / lam * factor, 1e-14))
    return cases
