"""Weights by tensor name, their one error, and the random-weights folder (no GPU)."""
import json
import os

import pytest
import torch

import braidinfer_amd as B
from braidinfer_amd.engine import DecoderModel
from braidinfer_amd.weights import (SafetensorsFolder, TensorSpec, load_tensors, write_safetensors,
                                    write_model_folder)
from conftest import TINY


def _specs(name="a"):
    cfg = B.MistralConfig.from_dict(TINY[name])
    return cfg, DecoderModel(B.spec_of(cfg)).weight_specs()


def test_container_round_trip(tmp_path):
    a = torch.randn(3, 5).bfloat16()
    b = torch.arange(7, dtype=torch.int32)
    c = torch.randn(4)
    write_safetensors(str(tmp_path / "model.safetensors"), [("a", a), ("b", b), ("c", c)])
    st = SafetensorsFolder(str(tmp_path))
    assert sorted(st.names()) == ["a", "b", "c"]
    assert torch.equal(st.tensor("a"), a) and torch.equal(st.tensor("b"), b) and torch.equal(st.tensor("c"), c)
    assert st.info("a") == (torch.bfloat16, (3, 5))


def test_the_same_file_reads_with_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    a = torch.randn(6, 2).bfloat16()
    write_safetensors(str(tmp_path / "model.safetensors"), [("w", a)])
    assert torch.equal(st.load_file(str(tmp_path / "model.safetensors"))["w"], a)


def test_random_folder_is_seeded_and_named_by_the_parts(tmp_path):
    cfg, specs = _specs("b")
    d1 = B.Engine.write_random_folder(str(tmp_path / "m1"), cfg, seed=5)
    d2 = B.Engine.write_random_folder(str(tmp_path / "m2"), cfg, seed=5)
    d3 = B.Engine.write_random_folder(str(tmp_path / "m3"), cfg, seed=6)
    assert json.load(open(os.path.join(d1, "config.json")))["architectures"] == ["MistralForCausalLM"]
    s1, s2, s3 = (SafetensorsFolder(d) for d in (d1, d2, d3))
    assert sorted(s1.names()) == sorted(s.name for s in specs)
    q = "model.layers.1.self_attn.q_proj.weight"
    assert s1.info(q) == (torch.bfloat16, (6 * 32, 96))
    assert torch.equal(s1.tensor(q), s2.tensor(q)) and not torch.equal(s1.tensor(q), s3.tensor(q))
    assert torch.all(s1.tensor("model.norm.weight") == 1)
    assert abs(s1.tensor(q).float().std().item() - 0.02) < 0.002
    assert B.config_from_folder(d1) == cfg


def test_dtypes_kept(tmp_path):
    specs = [TensorSpec("m16", (4, 8)), TensorSpec("m32", (4, 8)), TensorSpec("v", (8,), kind="vector"),
             TensorSpec("t", (5,), kind="int")]
    write_safetensors(str(tmp_path / "model.safetensors"),
                      [("m16", torch.randn(4, 8).bfloat16()), ("m32", torch.randn(4, 8)),
                       ("v", torch.randn(8).bfloat16()), ("t", torch.arange(5, dtype=torch.int64))])
    bf = load_tensors(str(tmp_path), specs, "cpu", torch.bfloat16)
    assert bf["m16"].dtype == torch.bfloat16      # bf16 stays bf16
    assert bf["m32"].dtype == torch.float32       # stored in 32-bit stays so
    assert bf["v"].dtype == torch.float32 and bf["t"].dtype == torch.int32
    f32 = load_tensors(str(tmp_path), specs, "cpu", torch.float32)
    assert f32["m16"].dtype == torch.float32 and torch.equal(f32["m16"], bf["m16"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg, specs = _specs("a")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=1)
    st = SafetensorsFolder(folder)
    tensors = {n: st.tensor(n).clone() for n in st.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.embed_tokens.weight"] = tensors["model.embed_tokens.weight"].to(torch.float16)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    with pytest.raises(B.WeightError) as ei:
        load_tensors(folder, specs, "cpu", torch.bfloat16)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert sorted(m[0] for m in e.mismatched) == ["model.embed_tokens.weight", "model.layers.0.self_attn.k_proj.weight"]
    msg = str(e)
    for word in ("up_proj", "model.norm.weight", "rotary_emb", "[32, 64]", "[16, 64]", "float16"):
        assert word in msg


def test_truncated_and_absent_files(tmp_path):
    with pytest.raises(B.WeightError, match="neither"):
        SafetensorsFolder(str(tmp_path))
    p = tmp_path / "model.safetensors"
    write_safetensors(str(p), [("a", torch.randn(100))])
    raw = p.read_bytes()
    p.write_bytes(raw[:-50])
    with pytest.raises(B.WeightError, match="truncated"):
        SafetensorsFolder(str(tmp_path))
    p.write_bytes(raw[:5])
    with pytest.raises(B.WeightError, match="truncated"):
        SafetensorsFolder(str(tmp_path))


def test_tied_head_needs_no_tensor_of_its_own():
    cfg, specs = _specs("c")
    names = [s.name for s in specs]
    assert "lm_head.weight" not in names and "model.embed_tokens.weight" in names
    cfg_a, specs_a = _specs("a")
    assert "lm_head.weight" in [s.name for s in specs_a]
