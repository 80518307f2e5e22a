"""Tiny configurations of the architecture that differ in every size and option, and
helpers that write them as model folders with random weights."""
from __future__ import annotations

import copy

from kappai_amd.config import config_from_dict
from kappai_amd.weights import write_random_model

# 4 layers conv/attention alternating, GQA 2:1, direct feed-forward width, tied head
TINY_A = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 64, "num_hidden_layers": 4,
    "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "intermediate_size": 192, "block_auto_adjust_ff_dim": False,
    "vocab_size": 256, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 4096,
}
INIT_A = dict(seed=0, std=0.02, norm_jitter=0.0)

# 6 layers, attention at 0, 3, 4, one kv head for three heads, width that is no power of two,
# auto-adjusted feed-forward width (480 -> 320), 4 taps with biases, untied head
TINY_B = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 96, "num_hidden_layers": 6,
    "layer_types": ["full_attention", "conv", "conv", "full_attention", "full_attention", "conv"],
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "intermediate_size": 480, "block_auto_adjust_ff_dim": True, "block_multiple_of": 64,
    "block_ffn_dim_multiplier": 1.0,
    "vocab_size": 512, "norm_eps": 1e-6, "rope_theta": 1000000.0,
    "conv_L_cache": 4, "conv_bias": True, "tie_embedding": False,
    "max_position_embeddings": 8192,
}
INIT_B = dict(seed=1, std=0.05, norm_jitter=0.1)

# 3 layers, as many kv heads as heads over two, head size 48 with heads * head size != width,
# a vocabulary and widths that are no powers of two, 2 taps
TINY_C = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 120, "num_hidden_layers": 3,
    "layer_types": ["full_attention", "conv", "full_attention"],
    "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48,
    "intermediate_size": 200, "block_auto_adjust_ff_dim": False,
    "vocab_size": 333, "norm_eps": 1e-4, "rope_theta": 50000.0,
    "conv_L_cache": 2, "conv_bias": False, "tie_embedding": False,
    "max_position_embeddings": 2048,
}
INIT_C = dict(seed=2, std=0.04, norm_jitter=0.05)

# 2 layers, a width, a feed-forward width and a vocabulary that are no multiples of 8 (the
# bfloat16 products then take their plain kernel), as many kv heads as heads, biases
TINY_D = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 100, "num_hidden_layers": 2, "layer_types": ["conv", "full_attention"],
    "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 16,
    "intermediate_size": 84, "block_auto_adjust_ff_dim": False,
    "vocab_size": 301, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": True, "tie_embedding": True,
    "max_position_embeddings": 1024,
}
INIT_D = dict(seed=3, std=0.05, norm_jitter=0.1)

# conv layers only: no paged cache at all, five taps
TINY_E = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 48, "num_hidden_layers": 3, "layer_types": ["conv", "conv", "conv"],
    "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 32,
    "intermediate_size": 112, "block_auto_adjust_ff_dim": False,
    "vocab_size": 200, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 5, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 1024,
}
INIT_E = dict(seed=4, std=0.05, norm_jitter=0.1)

# attention layers only, a single head of size 80 (wider than the model), no fixed state
TINY_F = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 56, "num_hidden_layers": 2,
    "layer_types": ["full_attention", "full_attention"],
    "num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 80,
    "intermediate_size": 144, "block_auto_adjust_ff_dim": False,
    "vocab_size": 150, "norm_eps": 1e-5, "rope_theta": 500000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": False,
    "max_position_embeddings": 1024,
}
INIT_F = dict(seed=5, std=0.05, norm_jitter=0.1)

# eighteen query heads on one kv head (more than the 16 columns of the matrix-core decode
# kernel: the other attention kernels run), attention first, a vocabulary that is a prime
TINY_G = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 72, "num_hidden_layers": 2, "layer_types": ["full_attention", "conv"],
    "num_attention_heads": 18, "num_key_value_heads": 1, "head_dim": 16,
    "intermediate_size": 96, "block_auto_adjust_ff_dim": False,
    "vocab_size": 257, "norm_eps": 1e-6, "rope_theta": 50000.0,
    "conv_L_cache": 2, "conv_bias": False, "tie_embedding": True,
    "max_position_embeddings": 1024,
}
INIT_G = dict(seed=6, std=0.05, norm_jitter=0.1)

# heads of 256, the largest size of the matrix-core attention kernels
TINY_H = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "hidden_size": 64, "num_hidden_layers": 2, "layer_types": ["conv", "full_attention"],
    "num_attention_heads": 2, "num_key_value_heads": 2, "head_dim": 256,
    "intermediate_size": 128, "block_auto_adjust_ff_dim": False,
    "vocab_size": 128, "norm_eps": 1e-5, "rope_theta": 10000.0,
    "conv_L_cache": 3, "conv_bias": False, "tie_embedding": False,
    "max_position_embeddings": 1024,
}
INIT_H = dict(seed=7, std=0.05, norm_jitter=0.1)

TINY = {"A": (TINY_A, INIT_A), "B": (TINY_B, INIT_B), "C": (TINY_C, INIT_C),
        "D": (TINY_D, INIT_D), "E": (TINY_E, INIT_E), "F": (TINY_F, INIT_F),
        "G": (TINY_G, INIT_G), "H": (TINY_H, INIT_H)}


def tiny_config(name: str) -> dict:
    return copy.deepcopy(TINY[name][0])


def write_tiny(name: str, folder, **overrides):
    cfg, init = TINY[name]
    init = {**init, **overrides}
    return write_random_model(folder, config_from_dict(copy.deepcopy(cfg)), **init)
