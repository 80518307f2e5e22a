"""Configuration of the LFM2 hybrid decoder (``Lfm2ForCausalLM``).

Field meanings follow kappai's ``model`` struct and its hybrid parameters
(src/model.h:179-259) and its checks at load (src/model.c:2309-2521, 278-586), with the
names of the architecture's own config.json keys.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Union

from .base import ConfigError, KeyReader, ModelConfig

ARCHITECTURE = "Lfm2ForCausalLM"

# kappai refuses heads wider than this (src/common.h:29, src/model.c:319-323); the
# attention kernels here are written for head sizes up to it.
MAX_HEAD_DIM = 512

_LAYER_TYPE_NAMES = {"conv": "conv", "full_attention": "attention", "attention": "attention"}


def adjusted_ff_dim(intermediate_size: int, auto_adjust: bool, multiple_of: int,
                    multiplier: Optional[float]) -> int:
    """Width of the SwiGLU hidden layer.  With ``block_auto_adjust_ff_dim`` the width is
    two thirds of ``intermediate_size``; when ``block_ffn_dim_multiplier`` is a number the
    width is multiplied by it and then rounded up to a multiple of ``block_multiple_of``
    (a multiplier of null leaves the two thirds as they are, unrounded); without
    ``block_auto_adjust_ff_dim`` it is ``intermediate_size`` itself.  (kappai reads the
    finished number, src/model.c:2329-2350.)"""
    if not auto_adjust:
        return intermediate_size
    f = (2 * intermediate_size) // 3
    if multiplier is None:
        return f
    f = int(multiplier * f)
    return multiple_of * ((f + multiple_of - 1) // multiple_of)


def _rope_theta(r: KeyReader) -> float:
    """``rope_theta``, at the top level or inside ``rope_parameters`` (where newer exports of the
    architecture's tools put it)."""
    nested = r.raw.get("rope_parameters")
    if r.raw.get("rope_theta") is None and isinstance(nested, dict) \
            and nested.get("rope_theta") is not None:
        return KeyReader(nested, r.where + ": rope_parameters").float("rope_theta")
    return r.float("rope_theta")


@dataclass
class Lfm2Config(ModelConfig):
    hidden_size: int = 0
    num_hidden_layers: int = 0
    layer_types: List[str] = None            # "conv" | "attention", one per layer
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    block_auto_adjust_ff_dim: bool = True
    block_multiple_of: int = 256
    block_ffn_dim_multiplier: Optional[float] = 1.0      # None: config.json says null
    vocab_size: int = 0
    norm_eps: float = 0.0
    rope_theta: float = 0.0
    conv_L_cache: int = 0
    conv_bias: bool = False
    tie_embedding: bool = True
    max_position_embeddings: int = 0         # 0: config.json names no longest sequence
    eos_token_id: Optional[Union[int, List[int]]] = None    # one id or several
    bos_token_id: Optional[int] = None
    pad_token_id: Optional[int] = None

    @property
    def ff_dim(self) -> int:
        return adjusted_ff_dim(self.intermediate_size, self.block_auto_adjust_ff_dim,
                               self.block_multiple_of, self.block_ffn_dim_multiplier)

    @property
    def attention_layers(self) -> List[int]:
        return [i for i, t in enumerate(self.layer_types) if t == "attention"]

    @property
    def conv_layers(self) -> List[int]:
        return [i for i, t in enumerate(self.layer_types) if t == "conv"]

    # ------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "Lfm2Config":
        r = KeyReader(raw)
        n_layers = r.int("num_hidden_layers")
        types = r.list("layer_types", None)
        if types is None:
            idxs = r.list("full_attn_idxs", None)
            if idxs is None:
                raise ConfigError("config.json: required key 'layer_types' is missing")
            types = ["full_attention" if i in idxs else "conv" for i in range(n_layers)]
        kinds = []
        for i, t in enumerate(types):
            if t not in _LAYER_TYPE_NAMES:
                raise ConfigError(f"config.json: layer_types[{i}] = {t!r}; known: "
                                  f"{', '.join(sorted(_LAYER_TYPE_NAMES))}")
            kinds.append(_LAYER_TYPE_NAMES[t])
        hidden = r.int("hidden_size")
        heads = r.int(("num_attention_heads", "num_heads"))
        head_dim = r.int("head_dim", None)
        if head_dim is None:
            if heads <= 0 or hidden % heads:
                raise ConfigError("config.json: 'head_dim' is absent and hidden_size is no "
                                  "multiple of num_attention_heads")
            head_dim = hidden // heads
        cfg = cls(
            architecture=ARCHITECTURE,
            hidden_size=hidden,
            num_hidden_layers=n_layers,
            layer_types=kinds,
            num_attention_heads=heads,
            num_key_value_heads=r.int("num_key_value_heads"),
            head_dim=head_dim,
            # the keys of the feed-forward width as the architecture's configuration files
            # define them: block_ff_dim, where present, is the number the rule starts from
            # (intermediate_size is its newer spelling); a file without the switch adjusts; a
            # file without the multiplier has 1.0, one that says null has none
            intermediate_size=r.int(("block_ff_dim", "intermediate_size")),
            block_auto_adjust_ff_dim=r.bool("block_auto_adjust_ff_dim", True),
            block_multiple_of=r.int("block_multiple_of", 256),
            block_ffn_dim_multiplier=(None if "block_ffn_dim_multiplier" in raw
                                      and raw["block_ffn_dim_multiplier"] is None
                                      else r.float("block_ffn_dim_multiplier", 1.0)),
            vocab_size=r.int("vocab_size"),
            norm_eps=r.float(("norm_eps", "block_norm_eps")),
            rope_theta=_rope_theta(r),
            conv_L_cache=r.int("conv_L_cache"),
            conv_bias=r.bool("conv_bias", False),
            tie_embedding=r.bool(("tie_embedding", "tie_word_embeddings"), True),
            max_position_embeddings=r.int("max_position_embeddings", 0),
            eos_token_id=r.int_or_ints("eos_token_id", None),
            bos_token_id=r.int("bos_token_id", None),
            pad_token_id=r.int("pad_token_id", None),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        """The reference's load-time checks (src/model.c:2368-2374 one entry per layer,
        :2491-2499 conv kernel >= 2 and kv heads >= 1, :319-323 head size) and those a
        grouped-query attention needs."""
        def need(cond, msg):
            if not cond:
                raise ConfigError("config.json: " + msg)

        need(self.num_hidden_layers >= 1, "num_hidden_layers must be at least 1")
        need(len(self.layer_types) == self.num_hidden_layers,
             f"layer_types has {len(self.layer_types)} entries for "
             f"{self.num_hidden_layers} layers")
        need(self.hidden_size >= 1, "hidden_size must be positive")
        need(self.vocab_size >= 1, "vocab_size must be positive")
        need(self.num_attention_heads >= 1, "num_attention_heads must be positive")
        need(self.num_key_value_heads >= 1, "num_key_value_heads must be at least 1")
        need(self.num_attention_heads % self.num_key_value_heads == 0,
             f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
             f"num_key_value_heads ({self.num_key_value_heads})")
        need(self.head_dim >= 2 and self.head_dim % 2 == 0,
             f"head_dim ({self.head_dim}) must be even for the rotation's pairs")
        need(self.head_dim <= MAX_HEAD_DIM, f"head_dim ({self.head_dim}) exceeds {MAX_HEAD_DIM}")
        need(self.head_dim % 8 == 0 or not self.attention_layers,
             f"head_dim ({self.head_dim}) must be a multiple of 8: the attention kernels read "
             "keys and values 8 at a time")
        need(self.conv_L_cache >= 2, f"conv_L_cache ({self.conv_L_cache}) must be at least 2")
        need(self.intermediate_size >= 1, "intermediate_size must be positive")
        need(self.block_multiple_of >= 1, "block_multiple_of must be positive")
        need(self.ff_dim >= 1, "the feed-forward width works out to zero")
        need(self.norm_eps > 0.0, "norm_eps must be positive")
        need(self.rope_theta > 0.0, "rope_theta must be positive")
        need(self.max_position_embeddings >= 0, "max_position_embeddings must not be negative")

    def to_dict(self) -> Dict[str, Any]:
        d = {
            "architectures": [ARCHITECTURE],
            "model_type": "lfm2",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "layer_types": ["conv" if t == "conv" else "full_attention" for t in self.layer_types],
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "block_auto_adjust_ff_dim": self.block_auto_adjust_ff_dim,
            "block_multiple_of": self.block_multiple_of,
            "vocab_size": self.vocab_size,
            "norm_eps": self.norm_eps,
            "rope_theta": self.rope_theta,
            "conv_L_cache": self.conv_L_cache,
            "conv_bias": self.conv_bias,
            "tie_embedding": self.tie_embedding,
            "max_position_embeddings": self.max_position_embeddings,
        }
        d["block_ffn_dim_multiplier"] = self.block_ffn_dim_multiplier     # null when None
        for k in ("eos_token_id", "bos_token_id", "pad_token_id"):
            if getattr(self, k) is not None:
                d[k] = getattr(self, k)
        return d
