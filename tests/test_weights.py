"""Weights: the container, loading by name, the one error that lists everything wrong, and
the random-weights mode."""
import json
import struct

import numpy as np
import pytest
import torch

from kappai_amd.models import load_model
from kappai_amd.weights import SafetensorsError, SafetensorsFile, WeightsError, write_safetensors
from plain import lfm2 as plain
from tiny import write_tiny


def test_container_round_trip(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.randn(7), "c": torch.arange(6, dtype=torch.int32)}
    write_safetensors(tmp_path / "x.safetensors", t, metadata={"k": "v"})
    with SafetensorsFile(tmp_path / "x.safetensors") as f:
        assert set(f.names()) == {"a", "b", "c"}
        for k, v in t.items():
            assert torch.equal(f.read(k), v)
    # the plain side's reader sees the same numbers
    mine = plain.read_safetensors(tmp_path / "x.safetensors")
    assert np.array_equal(mine["a"], t["a"].double().numpy())


def test_container_errors(tmp_path):
    p = tmp_path / "bad.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="shorter"):
        SafetensorsFile(p)
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="does not fit"):
        SafetensorsFile(p)
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="does not fit"):
        SafetensorsFile(p)


def test_random_model_is_reproducible_and_complete(tmp_path):
    a = write_tiny("B", tmp_path / "a")
    b = write_tiny("B", tmp_path / "b")
    c = write_tiny("B", tmp_path / "c", seed=5)
    fa, fb, fc = (plain.read_safetensors(d / "model.safetensors") for d in (a, b, c))
    assert fa.keys() == fb.keys()
    assert all(np.array_equal(fa[k], fb[k]) for k in fa)
    assert any(not np.array_equal(fa[k], fc[k]) for k in fa)
    cfg = json.loads((a / "config.json").read_text())
    assert cfg["architectures"] == ["Lfm2ForCausalLM"] and cfg["conv_L_cache"] == 4
    # untied head, conv biases, shapes from the configuration
    assert fa["lm_head.weight"].shape == (512, 96)
    assert fa["model.layers.1.conv.conv.weight"].shape == (96, 1, 4)
    assert fa["model.layers.1.conv.in_proj.bias"].shape == (288,)
    assert fa["model.layers.0.self_attn.k_proj.weight"].shape == (32, 96)
    assert fa["model.layers.0.feed_forward.w1.weight"].shape == (320, 96)
    assert "model.layers.0.conv.in_proj.weight" not in fa
    # norm weights 1 + N(0, 0.1); matrices N(0, 0.05)
    nw = fa["model.layers.2.operator_norm.weight"]
    assert 0.02 < nw.std() < 0.3 and abs(nw.mean() - 1) < 0.1
    assert 0.04 < fa["model.embed_tokens.weight"].std() < 0.06


def test_loads_on_cpu_and_keeps_dtypes(tmp_path):
    d = write_tiny("A", tmp_path / "m", vector_dtype=torch.float32)
    m16 = load_model(d, "bfloat16", "cpu")
    assert m16.embedding.table.dtype == torch.bfloat16
    assert m16.layers[0].mixer.in_proj.weight.dtype == torch.bfloat16
    assert m16.layers[0].mixer_norm.weight.dtype == torch.float32
    assert m16.head.linear.weight is m16.embedding.table          # tied
    m32 = load_model(d, "float32", "cpu")
    assert m32.layers[1].mixer.qkv.weight.dtype == torch.float32
    assert torch.equal(m32.embedding.table, m16.embedding.table.float())
    # a matrix stored in 32 bits stays so in a bfloat16 run
    f = SafetensorsFile(d / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    t["model.layers.0.conv.out_proj.weight"] = t["model.layers.0.conv.out_proj.weight"].float()
    write_safetensors(d / "model.safetensors", t)
    m = load_model(d, "bfloat16", "cpu")
    assert m.layers[0].mixer.out_proj.weight.dtype == torch.float32


def test_one_error_lists_everything(tmp_path):
    d = write_tiny("A", tmp_path / "m")
    f = SafetensorsFile(d / "model.safetensors")
    t = {n: f.read(n) for n in f.names()}
    f.close()
    del t["model.layers.1.self_attn.q_layernorm.weight"]
    del t["model.layers.2.conv.conv.weight"]
    t["model.layers.0.attention.wq"] = torch.zeros(2)
    t["lm_head.weight"] = torch.zeros(256, 64)            # tied model: not expected
    t["model.layers.3.feed_forward.w2.weight"] = torch.zeros(64, 100).to(torch.bfloat16)
    t["model.embedding_norm.weight"] = torch.zeros(63).to(torch.bfloat16)
    write_safetensors(d / "model.safetensors", t)
    with pytest.raises(WeightsError) as exc:
        load_model(d, "bfloat16", "cpu")
    e = exc.value
    assert e.missing == ["model.layers.1.self_attn.q_layernorm.weight",
                         "model.layers.2.conv.conv.weight"]
    assert e.unexpected == ["lm_head.weight", "model.layers.0.attention.wq"]
    assert len(e.wrong_shape) == 2
    msg = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (2)", "wrong shapes (2)",
                   "model.layers.3.feed_forward.w2.weight: file has [64, 100], model needs [64, 192]",
                   "model.embedding_norm.weight: file has [63], model needs [64]"):
        assert needle in msg, msg


def test_missing_file(tmp_path):
    d = write_tiny("A", tmp_path / "m")
    (d / "model.safetensors").unlink()
    with pytest.raises(WeightsError, match="no model.safetensors"):
        load_model(d, "float32", "cpu")


def test_container_refuses_overlapping_tensors(tmp_path):
    p = tmp_path / "overlap.safetensors"
    hdr = json.dumps({"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]},
                      "b": {"dtype": "F32", "shape": [4], "data_offsets": [8, 24]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 24)
    with pytest.raises(SafetensorsError, match="overlap"):
        SafetensorsFile(p)


@pytest.mark.parametrize("name", ["../model.safetensors", "/etc/passwd", "sub/x.safetensors", ".."])
def test_index_file_names_stay_inside_the_model_folder(tmp_path, name):
    d = write_tiny("A", tmp_path / "a")
    (d / "model.safetensors").rename(tmp_path / "model.safetensors")
    (d / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"model.embed_tokens.weight": name}}))
    with pytest.raises(WeightsError, match="plain file name inside the model folder"):
        load_model(d, "float32", device="cpu")
