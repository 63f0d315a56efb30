"""Configuration and registry (no GPU)."""
import json
import os

import pytest

import braidinfer_amd as B
from braidinfer_amd.config import (config_from_dict, config_from_folder, register_architecture,
                                   unregister_architecture, registered_architectures, spec_of)
from conftest import TINY


def test_reads_every_key():
    d = dict(TINY["b"], architectures=["MistralForCausalLM"], eos_token_id=[2, 7], bos_token_id=1)
    cfg = config_from_dict(d)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (3, 96, 6, 3)
    assert (cfg.head_dim, cfg.intermediate_size, cfg.vocab_size) == (32, 320, 384)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-6 and cfg.sliding_window == 8
    assert cfg.eos_token_id == (2, 7) and cfg.bos_token_id == 1 and cfg.tie_word_embeddings is False


def test_defaults_follow_the_reference_parser():
    # config.rs:233-277: kv heads = heads, head_dim = hidden / heads, eps 1e-5, theta 10000
    cfg = B.MistralConfig.from_dict(dict(num_hidden_layers=1, hidden_size=48, num_attention_heads=4,
                                         intermediate_size=64, vocab_size=50))
    assert cfg.num_key_value_heads == 4 and cfg.head_dim == 12
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 10000.0 and cfg.max_position_embeddings == 2048
    assert cfg.sliding_window is None and cfg.tie_word_embeddings is False and cfg.rope_pairing == "half"


def test_model_type_names_the_architecture_too():
    d = dict(TINY["a"], model_type="mistral")
    assert isinstance(config_from_dict(d), B.MistralConfig)


@pytest.mark.parametrize("bad, word", [
    (dict(num_attention_heads=5), "multiple"),
    (dict(head_dim=15), "even"),
    (dict(vocab_size=0), "positive"),
    (dict(sliding_window=0), "sliding_window"),
    (dict(rope_pairing="spiral"), "rope_pairing"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(num_hidden_layers="two"), "integer"),
    (dict(layer_types=["full_attention"]), "layer_types"),
])
def test_rejects_bad_values(bad, word):
    with pytest.raises(B.ConfigError, match=word):
        B.MistralConfig.from_dict(dict(TINY["a"], **bad))


def test_missing_key_is_named():
    d = dict(TINY["a"])
    del d["intermediate_size"]
    with pytest.raises(B.ConfigError, match="intermediate_size"):
        B.MistralConfig.from_dict(d)


def test_unknown_architecture_lists_the_known_ones():
    with pytest.raises(B.ConfigError, match="MistralForCausalLM"):
        config_from_dict({"architectures": ["NoSuchModel"]})
    with pytest.raises(B.ConfigError):
        config_from_dict({"hidden_size": 4})


def test_round_trip_through_a_folder(tmp_path):
    cfg = B.MistralConfig.from_dict(TINY["c"])
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg.to_dict(), f)
    assert config_from_folder(str(tmp_path)) == cfg
    with pytest.raises(B.ConfigError, match="config.json"):
        config_from_folder(str(tmp_path / "nowhere"))


def test_spec_holds_every_size_and_layer_choice():
    cfg = B.MistralConfig.from_dict(TINY["c"])
    spec = spec_of(cfg)
    assert len(spec.layers) == 4 and [e.layer for e in spec.schedule] == [0, 1, 2, 3]
    windows = [l.mixer.params["window"] for l in spec.layers]
    assert windows == [70, None, 70, None]
    m = spec.layers[0].mixer.params
    assert (m["num_heads"], m["num_kv_heads"], m["head_dim"], m["hidden_size"]) == (5, 1, 48, 100)
    assert spec.layers[0].feed_forward.params["intermediate_size"] == 172
    assert spec.positions["rope"].params == {"rotary_dim": 48, "theta": 500000.0, "pairing": "adjacent"}
    assert spec.lm_head.params["tied_to"] == "model.embed_tokens.weight"
    assert spec.final_norm.params["eps"] == 3e-6


def test_presets_are_the_benchmark_shapes():
    c = B.preset("mistral-7b-v0.3")
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            c.intermediate_size, c.vocab_size) == (32, 4096, 32, 8, 128, 14336, 32768)
    assert B.preset("mistral-7b-v0.1").sliding_window == 4096
    assert B.preset("mistral-small-24b").hidden_size == 5120
    with pytest.raises(B.ConfigError):
        B.preset("nothing")


def test_registering_another_architecture():
    class ToyConfig:
        architecture = "ToyForCausalLM"

        def __init__(self, d):
            self.d = d

        @classmethod
        def from_dict(cls, d):
            return cls(d)

    register_architecture("ToyForCausalLM", ToyConfig, lambda c: "spec of toy", model_type="toy")
    try:
        assert "ToyForCausalLM" in registered_architectures()
        cfg = config_from_dict({"architectures": ["ToyForCausalLM"], "x": 1})
        assert isinstance(cfg, ToyConfig) and spec_of(cfg) == "spec of toy"
        with pytest.raises(B.ConfigError, match="already"):
            register_architecture("ToyForCausalLM", ToyConfig, lambda c: None)
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in registered_architectures()


def test_a_head_size_no_kernel_takes_is_refused_when_the_configuration_is_read():
    d = dict(TINY["a"], head_dim=512)
    assert B.MistralConfig.from_dict(d).head_dim == 512
    with pytest.raises(B.ConfigError, match="head_dim 514"):
        B.MistralConfig.from_dict(dict(d, head_dim=514))
    with pytest.raises(B.ConfigError, match="head_dim 1024"):
        B.preset("tiny-a", head_dim=1024)


def test_stop_tokens_of_generation_config_json(tmp_path):
    from braidinfer_amd.config import generation_stop_tokens
    assert generation_stop_tokens(str(tmp_path)) == []
    (tmp_path / "generation_config.json").write_text('{"bos_token_id": 1, "eos_token_id": 2}')
    assert generation_stop_tokens(str(tmp_path)) == [2]
    (tmp_path / "generation_config.json").write_text('{"eos_token_id": [2, 7, 9]}')
    assert generation_stop_tokens(str(tmp_path)) == [2, 7, 9]
    (tmp_path / "generation_config.json").write_text('{"temperature": 0.7}')
    assert generation_stop_tokens(str(tmp_path)) == []
    (tmp_path / "generation_config.json").write_text('{"eos_token_id": "</s>"}')
    with pytest.raises(B.ConfigError, match="eos_token_id"):
        generation_stop_tokens(str(tmp_path))


def test_a_layer_names_its_norms_by_role_and_its_tensors_by_the_builder():
    spec = B.spec_of(B.MistralConfig.from_dict(TINY["a"]))
    layer = spec.layers[1]
    assert sorted(layer.norms) == ["feed_forward", "mixer"] and layer.block == "prenorm_residual"
    assert list(layer.names) == ["norm.mixer", "mixer", "norm.feed_forward", "feed_forward"]
    assert layer.name_of("norm.feed_forward") == "model.layers.1.post_attention_layernorm."
    with pytest.raises(KeyError):
        layer.name_of("norm.post_mixer")
    # nothing in the neutral description carries a checkpoint's names of its own
    bare = B.LayerSpec("p.")
    assert bare.names == {} and bare.norms == {} and bare.mixer is None


def test_scaled_rotary_frequencies_are_refused_not_ignored():
    B.MistralConfig.from_dict(dict(TINY["a"], rope_scaling=None))
    B.MistralConfig.from_dict(dict(TINY["a"], rope_scaling={"rope_type": "default"}))
    with pytest.raises(B.ConfigError, match="rope_scaling"):
        B.MistralConfig.from_dict(dict(TINY["a"], rope_scaling={"rope_type": "yarn", "factor": 4.0}))


def test_a_layer_spec_with_further_mixers_names_their_tensors_and_cache_units():
    from braidinfer_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from braidinfer_amd.engine import DecoderModel
    H = 32
    norm = PartSpec("rmsnorm", {"size": H, "eps": 1e-5})
    attn = lambda w: PartSpec("gqa_attention", {"hidden_size": H, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                                "window": w, "position": "rope"})
    names = {"mixer": "a.", "mixer.local": "b.", "norm.mixer": "n."}

    def spec(schedule, names=names):
        layer = LayerSpec("l.0.", attn(None), None, {"mixer": norm}, "prenorm_residual", names, more_mixers={"local": attn(4)})
        return ModelSpec(architecture="X", hidden_size=H, vocab_size=10, embedding=PartSpec("embedding", {"vocab_size": 10, "hidden_size": H}),
                         layers=[layer], schedule=schedule, final_norm=norm,
                         lm_head=PartSpec("lm_head", {"vocab_size": 10, "hidden_size": H, "tied_to": None}),
                         positions={"rope": PartSpec("rope", {"rotary_dim": 16, "theta": 1e4, "pairing": "half"})},
                         max_position_embeddings=64, embedding_prefix="e.", final_norm_prefix="f.", lm_head_prefix="h.")
    m = DecoderModel(spec([ScheduleEntry(0, 0, more_caches={"local": 1})]))
    got = [t.name for t in m.weight_specs()]
    assert "l.0.a.q_proj.weight" in got and "l.0.b.q_proj.weight" in got and got.index("l.0.a.o_proj.weight") < got.index("l.0.b.q_proj.weight")
    needs = m.cache_needs()
    assert sorted(needs) == [0, 1] and needs[0].window is None and needs[1].window == 4
    with pytest.raises(B.ConfigError, match="mixers the layer has not"):
        DecoderModel(spec([ScheduleEntry(0, 0, more_caches={"far": 1})]))
    with pytest.raises(B.ConfigError, match="no tensor-name piece"):
        DecoderModel(spec([ScheduleEntry(0, 0)], names={"mixer": "a.", "norm.mixer": "n."})).weight_specs()
