"""Bringing weights onto the GPU: the generator's kernel, the staging path, the arena."""
import numpy as np
import pytest
import torch

import braidinfer_amd as B
import plain_mistral as P
from braidinfer_amd import kernels as K
from braidinfer_amd.engine import DecoderModel
from braidinfer_amd.weights import (FolderTensors, RandomTensors, WeightArena, f32_to_bf16_bits, normal_f32, ones_f32,
                                    tensor_key)
from conftest import TINY

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("n,first", [(1, 0), (255, 0), (70001, 12345), (1 << 20, 2**33 + 7)])
def test_generator_kernel_gives_the_bits_of_the_numpy_form(n, first):
    key = tensor_key(2**50 + 3, 17)
    want = normal_f32(key, n, 0.02, first)
    got32 = torch.empty(n, dtype=torch.float32, device=DEV)
    K.random_normal(got32, key, 0.02, first)
    assert np.array_equal(got32.cpu().numpy().view(np.uint32), want.view(np.uint32))
    got16 = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    K.random_normal(got16, key, 0.02, first)
    assert np.array_equal(got16.cpu().view(torch.int16).numpy().view(np.uint16), f32_to_bf16_bits(want))
    ones = torch.empty(n, dtype=torch.float32, device=DEV)
    K.random_ones(ones, key, 0.3, first)
    assert np.array_equal(ones.cpu().numpy().view(np.uint32), ones_f32(key, n, 0.3, first).view(np.uint32))
    K.random_ones(ones, key, 0.0, first)
    assert bool((ones == 1).all())


@pytest.mark.parametrize("name", ["b", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_engine_and_random_folder_hold_the_same_model(tmp_path, name, dtype):
    """`Engine.random`, a folder of the same seed (one file, or shards brought through a
    staging buffer far smaller than a tensor) and the plain generator give equal logits:
    to the bit between the engines, within the dtype's bound against the plain forward."""
    cfg = B.MistralConfig.from_dict(TINY[name])
    d1 = B.Engine.write_random_folder(str(tmp_path / "one"), cfg, seed=21, std=0.08, vector_jitter=0.3)
    d2 = B.Engine.write_random_folder(str(tmp_path / "many"), cfg, seed=21, std=0.08, vector_jitter=0.3,
                                      shard_bytes=50_000, device=DEV)
    rng = np.random.default_rng(4)
    toks = [int(t) for t in rng.integers(0, cfg.vocab_size, 40)]
    outs = []
    for make in (lambda: B.Engine.random(cfg, seed=21, std=0.08, vector_jitter=0.3, dtype=dtype, max_tokens=256),
                 lambda: B.Engine.from_folder(d1, dtype=dtype, max_tokens=256),
                 lambda: B.Engine.from_folder(d2, dtype=dtype, max_tokens=256)):
        eng = make()
        s = eng.alloc_slot()
        outs.append(eng.step([B.StepEntry(s, toks, list(range(len(toks))))]).cpu().numpy())
        assert eng.load_profile is not None and "LOAD PROFILE" in eng.load_profile.line()
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    pc, _ = P.read_folder(d1)
    want = P.forward(pc, P.random_weights(pc, 21, 0.08, 0.3), toks)
    tol = 1e-4 if dtype == "float32" else 3e-2
    assert np.abs(outs[0] - want).max() <= tol * np.abs(want).max()


def test_what_the_parts_keep_lies_in_one_arena(tmp_path):
    cfg = B.MistralConfig.from_dict(dict(TINY["a"], hidden_size=1024, intermediate_size=4096, num_attention_heads=8,
                                         num_key_value_heads=2, head_dim=128, vocab_size=9000))
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=2, device=DEV)
    for eng in (B.Engine.from_folder(folder, max_tokens=128), B.Engine.random(cfg, seed=2, max_tokens=128)):
        arena = eng.rt.arena
        kept = [eng.model.embedding.weight, eng.model.lm_head.weight, eng.model.final_norm.weight]
        for layer in eng.model.layers:
            kept += [layer.mixer.w_qkv, layer.mixer.w_o, layer.feed_forward.w_gu, layer.feed_forward.w_d,
                     layer.mixer_norm.weight, layer.ffn_norm.weight]
        assert all(arena.holds(t) for t in kept)
        assert eng.model.lm_head.weight.dim() == 4 and eng.model.layers[0].feed_forward.w_gu.dim() == 4   # blocked in place
        assert arena.spilled == 0 and arena.used <= arena.buf.numel()
        assert eng.load_profile.arena_used == arena.used
        # no two kept tensors overlap
        spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * t.element_size()) for t in kept)
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))


def test_staging_in_pieces_brings_every_byte(tmp_path):
    """A tensor far larger than the staging buffers, with a size that is no multiple of
    them, arrives whole and in order; so does a tensor pulled twice."""
    cfg = B.MistralConfig.from_dict(dict(TINY["a"], vocab_size=5003, hidden_size=1000, head_dim=250))
    folder = B.Engine.write_random_folder(str(tmp_path / "m"), cfg, seed=8, std=0.05)
    specs = DecoderModel(B.spec_of(cfg)).weight_specs()
    src = FolderTensors(folder, specs, DEV, torch.bfloat16, staging_bytes=1 << 16, read_threads=3)
    ref = RandomTensors(specs, 8, "cpu", torch.bfloat16, std=0.05)
    for s in specs + specs[:3]:
        got = src[s.name]
        assert got.device.type == "cuda" and torch.equal(got.cpu(), ref[s.name]), s.name
    prof = src.finish()
    assert prof.file_bytes >= sum(2 * int(np.prod(s.shape)) for s in specs) and prof.seconds > 0
    # the 32-bit path widens on the device
    src32 = FolderTensors(folder, specs, DEV, torch.float32, staging_bytes=1 << 16)
    w = src32["model.embed_tokens.weight"]
    assert w.dtype == torch.float32 and torch.equal(w.cpu(), ref["model.embed_tokens.weight"].float())
    src32.finish()


def test_an_arena_too_small_spills_instead_of_failing():
    a = WeightArena(DEV, 1024)
    x = a.empty((100,), torch.float32)
    y = a.empty((1000,), torch.float32)
    assert a.holds(x) and not a.holds(y) and a.spilled == 4000
