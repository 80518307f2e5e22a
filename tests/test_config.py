"""Configuration: typed reading of config.json keys, the registry, and validation."""
import copy
import json

import pytest

from kappai_amd.config import (ConfigError, Lfm2Config, adjusted_ff_dim, config_from_dict,
                               known_architectures, load_config, lookup_architecture)
from plain import lfm2 as plain
from tiny import TINY_A, TINY_B, TINY_C

LFM2_1_2B = {
    "architectures": ["Lfm2ForCausalLM"], "hidden_size": 2048, "num_hidden_layers": 16,
    "layer_types": ["conv", "conv", "full_attention", "conv", "conv", "full_attention", "conv",
                    "conv", "full_attention", "conv", "full_attention", "conv", "full_attention",
                    "conv", "full_attention", "conv"],
    "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 12288,
    "block_auto_adjust_ff_dim": True, "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0,
    "vocab_size": 65536, "norm_eps": 1e-5, "rope_theta": 1000000.0, "conv_L_cache": 3,
    "conv_bias": False, "tie_embedding": True, "max_position_embeddings": 128000,
}


def test_feed_forward_width_examples():
    # the worked examples of the architecture's published sizes
    assert adjusted_ff_dim(12288, True, 256, 1.0) == 8192
    assert adjusted_ff_dim(6656, True, 256, 1.0) == 4608
    assert adjusted_ff_dim(10752, True, 256, 1.0) == 7168
    assert adjusted_ff_dim(480, True, 64, 1.0) == 320
    assert adjusted_ff_dim(192, False, 256, None) == 192
    assert adjusted_ff_dim(480, True, 64, None) == 320
    assert adjusted_ff_dim(500, True, 64, None) == 333      # no multiplier: not rounded either
    assert adjusted_ff_dim(500, True, 64, 1.0) == 384
    assert adjusted_ff_dim(500, True, 64, 1.5) == 512       # int(1.5 * 333) = 499
    for cfg in (TINY_A, TINY_B, TINY_C, LFM2_1_2B):
        assert config_from_dict(copy.deepcopy(cfg)).ff_dim == plain.feed_forward_width(cfg)


def test_feed_forward_width_when_keys_are_absent():
    """A config.json without the switch adjusts (two thirds), without the multiplier has 1.0
    (so the width is rounded), with a multiplier of null is not rounded, and ``block_ff_dim``
    is the number the rule starts from when both spellings are there.  Product and plain
    implementation are held to the same four cases."""
    base = copy.deepcopy(TINY_A)
    for k in ("block_auto_adjust_ff_dim", "block_multiple_of", "block_ffn_dim_multiplier"):
        base.pop(k, None)
    base["intermediate_size"] = 500
    cases = [({}, 512),                                              # 333 -> next 256
             ({"block_multiple_of": 64}, 384),
             ({"block_multiple_of": 64, "block_ffn_dim_multiplier": None}, 333),
             ({"block_auto_adjust_ff_dim": False}, 500),
             ({"block_ff_dim": 300, "block_multiple_of": 8}, 200),
             ({"block_ff_dim": 300, "block_auto_adjust_ff_dim": False}, 300)]
    for extra, want in cases:
        raw = dict(copy.deepcopy(base), **extra)
        cfg = config_from_dict(copy.deepcopy(raw))
        assert cfg.ff_dim == want == plain.feed_forward_width(raw), (extra, cfg.ff_dim)
        again = config_from_dict(cfg.to_dict())
        assert again.ff_dim == want and again == cfg


def test_named_shapes():
    """The shapes that --random-weights and the benchmark know by name: the sizes of the
    architecture's three published models and the two tiny configurations of the tests."""
    from kappai_amd.config import SHAPES, named_shape
    for name, ff, layers, attention in (
            ("lfm2-1.2b", 8192, 16, [2, 5, 8, 10, 12, 14]),
            ("lfm2-350m", 4608, 16, [2, 5, 8, 10, 12, 14]),
            ("LFM2-2.6B", 7168, 30, [2, 6, 10, 14, 18, 21, 24, 27]),
            ("tiny-a", 192, 4, [1, 3]), ("tiny-b", 320, 6, [0, 3, 4])):
        cfg = config_from_dict(named_shape(name))
        assert (cfg.ff_dim, cfg.num_hidden_layers, cfg.attention_layers) == (ff, layers, attention)
    assert named_shape("tiny-a") == TINY_A and named_shape("tiny-b") == TINY_B
    named_shape("tiny-a")["hidden_size"] = 1          # a copy: the table is not changed
    assert SHAPES["tiny-a"]["hidden_size"] == 64
    with pytest.raises(KeyError, match="known: lfm2-1.2b"):
        named_shape("lfm2-7b")


def test_lfm2_1_2b_shape():
    c = config_from_dict(copy.deepcopy(LFM2_1_2B))
    assert isinstance(c, Lfm2Config)
    assert c.head_dim == 64 and c.ff_dim == 8192
    assert c.attention_layers == [2, 5, 8, 10, 12, 14] and len(c.conv_layers) == 10
    again = config_from_dict(c.to_dict())
    assert again == c


def test_full_attn_idxs_form():
    raw = copy.deepcopy(LFM2_1_2B)
    del raw["layer_types"]
    raw["full_attn_idxs"] = [2, 5, 8, 10, 12, 14]
    assert config_from_dict(raw).attention_layers == [2, 5, 8, 10, 12, 14]


def test_registry():
    assert "Lfm2ForCausalLM" in known_architectures()
    assert lookup_architecture("Lfm2ForCausalLM").config_cls is Lfm2Config
    with pytest.raises(ConfigError, match="unrecognized architecture 'LlamaForCausalLM'.*Lfm2"):
        config_from_dict({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({"hidden_size": 8})


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads",
                                 "num_key_value_heads", "intermediate_size", "vocab_size",
                                 "norm_eps", "rope_theta", "conv_L_cache"])
def test_required_keys(key):
    raw = copy.deepcopy(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


def test_other_spellings_of_the_same_keys():
    """Exports of the architecture's own tools have named some keys differently over time
    (block_ff_dim, block_norm_eps, num_heads, tie_word_embeddings, rope_parameters.rope_theta);
    the key of today wins where both are there (but ``block_ff_dim``, which the width rule starts from).  A config without max_position_embeddings
    names no longest sequence."""
    raw = copy.deepcopy(TINY_A)
    want = config_from_dict(copy.deepcopy(raw))
    for old_key, new_key in (("intermediate_size", "block_ff_dim"), ("norm_eps", "block_norm_eps"),
                             ("num_attention_heads", "num_heads"),
                             ("tie_embedding", "tie_word_embeddings")):
        raw[new_key] = raw.pop(old_key)
    raw["rope_parameters"] = {"rope_theta": raw.pop("rope_theta"), "rope_type": "default"}
    del raw["max_position_embeddings"]
    got = config_from_dict(copy.deepcopy(raw))
    assert got.max_position_embeddings == 0
    got.max_position_embeddings = want.max_position_embeddings
    assert got == want
    raw["norm_eps"], raw["block_norm_eps"] = 1e-3, 1e-7
    assert config_from_dict(raw).norm_eps == 1e-3


@pytest.mark.parametrize("change,match", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"num_key_value_heads": 0}, "at least 1"),
    ({"conv_L_cache": 1}, "conv_L_cache"),
    ({"head_dim": 15}, "even"),
    ({"head_dim": 1024}, "exceeds"),
    ({"head_dim": 18}, "multiple of 8"),
    ({"layer_types": ["conv"]}, "layer_types has 1 entries for 4 layers"),
    ({"layer_types": ["conv", "mamba", "conv", "full_attention"]}, "layer_types\\[1\\]"),
    ({"hidden_size": "64"}, "integer"),
    ({"conv_bias": 1}, "true or false"),
    ({"norm_eps": 0.0}, "norm_eps"),
])
def test_rejected(change, match):
    raw = copy.deepcopy(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError, match=match):
        config_from_dict(raw)


def test_end_of_sequence_ids_one_or_several():
    """Checkpoints write ``eos_token_id`` as one id or as a list; both are kept as written, and
    anything else is refused."""
    raw = copy.deepcopy(LFM2_1_2B)
    assert config_from_dict(raw).eos_token_id is None
    raw["eos_token_id"] = 7
    cfg = config_from_dict(raw)
    assert cfg.eos_token_id == 7 and cfg.to_dict()["eos_token_id"] == 7
    raw["eos_token_id"] = [7, 2]
    cfg = config_from_dict(raw)
    assert cfg.eos_token_id == [7, 2] and cfg.to_dict()["eos_token_id"] == [7, 2]
    for bad in ("7", [7, "2"], 7.5, [True]):
        raw["eos_token_id"] = bad
        with pytest.raises(ConfigError, match="eos_token_id"):
            config_from_dict(raw)


def test_head_dim_defaults_to_width_over_heads():
    raw = copy.deepcopy(TINY_A)
    del raw["head_dim"]
    assert config_from_dict(raw).head_dim == 16
    raw["num_attention_heads"] = 5
    raw["num_key_value_heads"] = 5
    with pytest.raises(ConfigError, match="head_dim"):
        config_from_dict(raw)


def test_load_config_errors(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    assert load_config(tmp_path).hidden_size == 96
