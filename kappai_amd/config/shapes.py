"""Named configurations for the random-weights mode: config.json contents by name.

These are data, not defaults: no part of the engine reads a size from here.  ``--random-weights
NAME`` writes a model folder of that shape; the benchmark uses the same dictionaries.  The sizes
are those of the architecture's published models (the three LFM2 shapes) and of two tiny
configurations that differ in every size and option.
"""
from __future__ import annotations

import copy
from typing import Dict


def _lfm2(hidden, layers, attention_at, heads, kv_heads, intermediate, **more) -> dict:
    raw = {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": hidden,
        "num_hidden_layers": layers,
        "layer_types": ["full_attention" if i in attention_at else "conv" for i in range(layers)],
        "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": 64,
        "intermediate_size": intermediate, "block_auto_adjust_ff_dim": True,
        "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0, "vocab_size": 65536,
        "norm_eps": 1e-5, "rope_theta": 1000000.0, "conv_L_cache": 3, "conv_bias": False,
        "tie_embedding": True, "max_position_embeddings": 128000,
    }
    raw.update(more)
    return raw


SHAPES: Dict[str, dict] = {
    # 16 layers, attention at 2, 5, 8, 10, 12, 14; feed-forward 12288 -> 8192
    "lfm2-1.2b": _lfm2(2048, 16, (2, 5, 8, 10, 12, 14), 32, 8, 12288),
    # the same pattern at half the width; feed-forward 6656 -> 4608
    "lfm2-350m": _lfm2(1024, 16, (2, 5, 8, 10, 12, 14), 16, 8, 6656),
    # 30 layers, attention at 2, 6, 10, 14, 18, 21, 24, 27; feed-forward 10752 -> 7168
    "lfm2-2.6b": _lfm2(2048, 30, (2, 6, 10, 14, 18, 21, 24, 27), 32, 8, 10752),
    # 4 layers conv/attention alternating, two kv heads for four heads, tied head
    "tiny-a": {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 64,
        "num_hidden_layers": 4,
        "layer_types": ["conv", "full_attention", "conv", "full_attention"],
        "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
        "intermediate_size": 192, "block_auto_adjust_ff_dim": False, "vocab_size": 256,
        "norm_eps": 1e-5, "rope_theta": 10000.0, "conv_L_cache": 3, "conv_bias": False,
        "tie_embedding": True, "max_position_embeddings": 4096,
    },
    # 6 layers, attention at 0, 3, 4, one kv head for three heads, a width that is no power of two,
    # adjusted feed-forward width (480 -> 320), 4 taps with biases, untied head
    "tiny-b": {
        "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2", "hidden_size": 96,
        "num_hidden_layers": 6,
        "layer_types": ["full_attention", "conv", "conv", "full_attention", "full_attention",
                        "conv"],
        "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
        "intermediate_size": 480, "block_auto_adjust_ff_dim": True, "block_multiple_of": 64,
        "block_ffn_dim_multiplier": 1.0, "vocab_size": 512, "norm_eps": 1e-6,
        "rope_theta": 1000000.0, "conv_L_cache": 4, "conv_bias": True, "tie_embedding": False,
        "max_position_embeddings": 8192,
    },
}


def named_shape(name: str) -> dict:
    """A copy of the configuration called ``name`` (any case), or a ``KeyError`` naming them all."""
    key = name.strip().lower()
    if key not in SHAPES:
        raise KeyError(f"no shape named {name!r}; known: {', '.join(sorted(SHAPES))}")
    return copy.deepcopy(SHAPES[key])
