"""The LFM2 hybrid decoder put together from parts (kappai: src/models/lfm.c:7-62,
registered at :155-164; registry entry src/arch.c:74-82: qk-norm, rotate-half rotation,
hybrid with short convolutions).

Layer i is a conv layer or an attention layer as ``layer_types`` says; both kinds share
the pre-norm arrangement and the SwiGLU feed-forward.  Tensor names are those of the
architecture's checkpoints.
"""
from __future__ import annotations

import torch

from ..config.base import register_architecture
from ..config.lfm2 import ARCHITECTURE, Lfm2Config
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .base import Model


def build_lfm2(config: Lfm2Config, dtype: torch.dtype) -> Model:
    width = config.hidden_size
    rotary = make_part("position_encoding", "rotary", head_dim=config.head_dim,
                       theta=config.rope_theta, pairing="half")
    layers = []
    for i, kind in enumerate(config.layer_types):
        p = f"model.layers.{i}."
        if kind == "conv":
            mixer = make_part("mixer", "conv", prefix=p + "conv.", width=width,
                              kernel_size=config.conv_L_cache, dtype=dtype, bias=config.conv_bias)
        else:
            mixer = make_part("mixer", "attention", prefix=p + "self_attn.", width=width,
                              num_heads=config.num_attention_heads,
                              num_kv_heads=config.num_key_value_heads, head_dim=config.head_dim,
                              dtype=dtype, position=rotary, qk_norm_eps=config.norm_eps)
        layers.append(make_part(
            "block", "pre_norm",
            mixer_norm=make_part("norm", "rmsnorm", name=p + "operator_norm", width=width,
                                 eps=config.norm_eps, dtype=dtype),
            mixer=mixer,
            ffn_norm=make_part("norm", "rmsnorm", name=p + "ffn_norm", width=width,
                               eps=config.norm_eps, dtype=dtype),
            feed_forward=make_part("feed_forward", "swiglu", prefix=p + "feed_forward.",
                                   width=width, hidden=config.ff_dim, dtype=dtype)))
    embedding = TokenEmbedding("model.embed_tokens", config.vocab_size, width)
    final_norm = make_part("norm", "rmsnorm", name="model.embedding_norm", width=width,
                           eps=config.norm_eps, dtype=dtype)
    head = OutputHead("lm_head", config.vocab_size, width,
                      tied_to=embedding if config.tie_embedding else None)
    return Model(config, dtype, embedding, layers, final_norm, head)


register_architecture(ARCHITECTURE, Lfm2Config, build_lfm2)
