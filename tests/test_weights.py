"""Weights by tensor name, their one error, and the random-weights folder (no GPU)."""
import json
import os

import pytest
import torch

import braidinfer_amd as B
from braidinfer_amd.engine import DecoderModel
import numpy as np

import plain_mistral as P
from braidinfer_amd.weights import (INDEX_NAME, SafetensorsFolder, SafetensorsWriter, TensorSpec, load_tensors,
                                    normal_f32, tensor_key, write_safetensors, write_model_folder)
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


def test_random_weights_are_the_generator_defined_in_the_text(tmp_path):
    """The folder's bytes equal what the plain implementation computes with Python integers
    from the generator's definition: seed, tensor index, element index, nothing else."""
    for name, seed, std, jitter in (("a", 3, 0.08, 0.3), ("c", 2**40 + 5, 0.02, 0.0)):
        cfg, specs = _specs(name)
        d = B.Engine.write_random_folder(str(tmp_path / name), cfg, seed=seed, std=std, vector_jitter=jitter)
        pc, pw = P.read_folder(d)
        assert [n for n, _ in P.tensor_names(pc)] == [s.name for s in specs]
        want = P.random_weights(pc, seed, std, jitter)
        assert sorted(want) == sorted(pw)
        for n in want:
            assert np.array_equal(want[n].view(np.uint32), pw[n].view(np.uint32)), n
    if True:      # moments of a million values
        x = normal_f32(tensor_key(9, 4), 1 << 20, 1.0)
        assert abs(float(x.mean())) < 4e-3 and abs(float(x.std()) - 1.0) < 4e-3
        # a sum of twelve uniform numbers: kurtosis -0.1, so 0.678 of the mass within one std where the
        # normal has 0.6827; within two, 0.9545 either way
        assert abs(float((np.abs(x) < 1.0).mean()) - 0.6827) < 6e-3 and abs(float((np.abs(x) < 2.0).mean()) - 0.9545) < 3e-3
        # any piece of a tensor is the same numbers as that piece of the whole
        assert np.array_equal(normal_f32(tensor_key(9, 4), 1000, 1.0, first=777), x[777:1777])
        assert not np.array_equal(normal_f32(tensor_key(9, 5), 1000, 1.0), x[:1000])


def test_the_writer_puts_the_header_first_and_takes_tensors_in_order(tmp_path):
    p = str(tmp_path / "model.safetensors")
    a, b = torch.randn(3, 4).bfloat16(), torch.arange(5, dtype=torch.int32)
    with SafetensorsWriter(p, [("a", a.dtype, tuple(a.shape)), ("b", b.dtype, tuple(b.shape))]) as w:
        size_after_header = os.path.getsize(p) if w._f.flush() is None else 0
        w.write("a", a)
        w.write("b", b)
    assert os.path.getsize(p) == size_after_header + a.numel() * 2 + b.numel() * 4
    st = SafetensorsFolder(str(tmp_path))
    assert torch.equal(st.tensor("a"), a) and torch.equal(st.tensor("b"), b)
    with pytest.raises(B.WeightError, match="expected a"):
        with SafetensorsWriter(p, [("a", a.dtype, tuple(a.shape)), ("b", b.dtype, tuple(b.shape))]) as w:
            w.write("b", b)
    with pytest.raises(B.WeightError, match="never written"):
        with SafetensorsWriter(p, [("a", a.dtype, tuple(a.shape)), ("b", b.dtype, tuple(b.shape))]) as w:
            w.write("a", a)


def test_a_folder_in_shards_reads_like_one_file(tmp_path):
    cfg, specs = _specs("b")
    one = B.Engine.write_random_folder(str(tmp_path / "one"), cfg, seed=5, std=0.05)
    many = B.Engine.write_random_folder(str(tmp_path / "many"), cfg, seed=5, std=0.05, shard_bytes=60_000)
    files = sorted(f for f in os.listdir(many) if f.endswith(".safetensors"))
    assert len(files) >= 3 and "model.safetensors" not in files and os.path.isfile(os.path.join(many, INDEX_NAME))
    assert files[0] == f"model-00001-of-{len(files):05d}.safetensors"
    index = json.load(open(os.path.join(many, INDEX_NAME)))
    assert sorted(index["weight_map"]) == sorted(s.name for s in specs) and set(index["weight_map"].values()) == set(files)
    assert index["metadata"]["total_size"] == sum(2 * int(np.prod(s.shape)) for s in specs)
    a = load_tensors(one, specs, "cpu", torch.bfloat16)
    b = load_tensors(many, specs, "cpu", torch.bfloat16)
    assert all(torch.equal(a[n], b[n]) for n in a) and len(a) == len(b) == len(specs)
    (_, pa), (_, pb) = P.read_folder(one), P.read_folder(many)
    assert all(np.array_equal(pa[n], pb[n]) for n in pa) and sorted(pa) == sorted(pb)


def test_shard_errors(tmp_path):
    cfg, specs = _specs("a")
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=1, shard_bytes=30_000)
    files = sorted(f for f in os.listdir(folder) if f.endswith(".safetensors"))
    index_path = os.path.join(folder, INDEX_NAME)
    index = json.load(open(index_path))
    # a tensor that two files hold
    st = SafetensorsFolder(folder)
    first = {n: st.tensor(n).clone() for n in st.files[0].names()}
    dup = st.files[1].names()[0]
    first[dup] = st.tensor(dup).clone()
    del st
    write_safetensors(os.path.join(folder, files[0]), first.items())
    with pytest.raises(B.WeightError, match="appears in two files") as ei:
        load_tensors(folder, specs, "cpu", torch.bfloat16)
    assert dup in str(ei.value)
    del first[dup]
    write_safetensors(os.path.join(folder, files[0]), first.items())
    load_tensors(folder, specs, "cpu", torch.bfloat16)
    # the index places a tensor in a file that does not hold it
    moved = dict(index, weight_map=dict(index["weight_map"]))
    moved["weight_map"][dup] = files[0]
    json.dump(moved, open(index_path, "w"))
    with pytest.raises(B.WeightError, match="do not hold them"):
        SafetensorsFolder(folder)
    # a tensor the index forgot is still found in its file, one that no file holds is missing
    json.dump(index, open(index_path, "w"))
    os.remove(os.path.join(folder, files[-1]))
    with pytest.raises(B.WeightError, match="not there") as ei:
        load_tensors(folder, specs, "cpu", torch.bfloat16)
    assert files[-1] in str(ei.value)
    json.dump({"weight_map": []}, open(index_path, "w"))
    with pytest.raises(B.WeightError, match="weight_map"):
        SafetensorsFolder(folder)
    # a file name that leads out of the folder is refused before anything is opened
    for elsewhere in ("../m2/" + files[0], os.path.join(str(tmp_path), "m", files[0]), "sub/" + files[0]):
        json.dump({"weight_map": dict(index["weight_map"], **{dup: elsewhere})}, open(index_path, "w"))
        with pytest.raises(B.WeightError, match="outside the model folder"):
            SafetensorsFolder(folder)


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
