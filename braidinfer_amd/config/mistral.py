"""Typed configuration of `MistralForCausalLM` and its translation into parts.

Keys and defaults follow the reference's parser where it has them
(crates/braidinfer-runtime/src/config.rs:208-277): `num_key_value_heads` defaults to
the number of heads (:233-246), `head_dim` to hidden/heads (:247), `rms_norm_eps` to
1e-5 (:249-252), `rope_theta` to 10000 (:253-260), `max_position_embeddings` to 2048
(:269-272).  Two deliberate differences: `tie_word_embeddings` defaults to false (the
reference defaults it to true, config.rs:273-277, which silently reuses the embedding
for checkpoints that omit the key), and `sliding_window` is read (the reference never
parses it, config.rs:416).
"""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional, Tuple

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, default_schedule, prenorm_layer

ARCHITECTURE = "MistralForCausalLM"


def _int(d, key, default=None, required=False):
    if key not in d or d[key] is None:
        if required:
            raise ConfigError(f"config.json: missing required key '{key}'")
        return default
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int):
        raise ConfigError(f"config.json: '{key}' must be an integer, found {v!r}")
    return v


def _float(d, key, default):
    if key not in d or d[key] is None:
        return default
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' must be a number, found {v!r}")
    return float(v)


@dataclass(frozen=True)
class MistralConfig:
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    sliding_window: Optional[int] = None
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 2048
    # "half": element i pairs with i + head_dim/2 (the layout of MistralForCausalLM
    # checkpoints); "adjacent": (2i, 2i+1) as the reference's kernel rotates
    # (kernels/megakernel_ops.hip:2019-2030).
    rope_pairing: str = "half"
    # per layer "full_attention" | "sliding_attention"; None = all layers use
    # `sliding_window` when it is set
    layer_types: Optional[Tuple[str, ...]] = None
    eos_token_id: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    hidden_act: str = "silu"

    architecture = ARCHITECTURE

    # ---- reading -------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MistralConfig":
        heads = _int(d, "num_attention_heads", required=True)
        hidden = _int(d, "hidden_size", required=True)
        if heads is not None and heads <= 0:
            raise ConfigError(f"config.json: num_attention_heads must be positive, found {heads}")
        head_dim = _int(d, "head_dim", default=None)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: no head_dim given and hidden_size {hidden} is not a "
                    f"multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"config.json: eos_token_id must be an integer or a list, found {eos!r}")
        lt = d.get("layer_types")
        if lt is not None:
            if not isinstance(lt, (list, tuple)) or not all(isinstance(t, str) for t in lt):
                raise ConfigError("config.json: layer_types must be a list of strings")
            lt = tuple(lt)
        # rotary frequencies are the plain ones (the reference has no scaling of any kind either,
        # config.rs:253-272): a configuration that asks for scaled ones is refused, not run unscaled
        scaling = d.get("rope_scaling")
        if scaling not in (None, {}) and not (isinstance(scaling, dict) and scaling.get("rope_type", scaling.get("type")) in (None, "default")):
            raise ConfigError(f"config.json: rope_scaling {scaling!r} is not supported (plain rotary frequencies only)")
        tie = d.get("tie_word_embeddings", False)
        if not isinstance(tie, bool):
            raise ConfigError(f"config.json: tie_word_embeddings must be a boolean, found {tie!r}")
        cfg = cls(
            num_hidden_layers=_int(d, "num_hidden_layers", required=True),
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=_int(d, "num_key_value_heads", default=heads),
            head_dim=head_dim,
            intermediate_size=_int(d, "intermediate_size", required=True),
            vocab_size=_int(d, "vocab_size", required=True),
            rope_theta=_float(d, "rope_theta", 10000.0),
            rms_norm_eps=_float(d, "rms_norm_eps", 1e-5),
            sliding_window=_int(d, "sliding_window", default=None),
            tie_word_embeddings=tie,
            max_position_embeddings=_int(d, "max_position_embeddings", default=2048),
            rope_pairing=d.get("rope_pairing", "half"),
            layer_types=lt,
            eos_token_id=eos_ids,
            bos_token_id=_int(d, "bos_token_id", default=None),
            hidden_act=d.get("hidden_act", "silu"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in ("num_hidden_layers", "hidden_size", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "vocab_size",
                     "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: {name} must be positive, found {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        from ..parts.attention import MAX_HEAD_DIM      # the attention part's own limit, refused here already
        if self.head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: head_dim {self.head_dim} is beyond the largest head size any attention "
                              f"kernel of this library takes ({MAX_HEAD_DIM})")
        if self.sliding_window is not None and self.sliding_window <= 0:
            raise ConfigError(f"config.json: sliding_window must be positive or null, found {self.sliding_window}")
        if self.rope_pairing not in ("half", "adjacent"):
            raise ConfigError(f"config.json: rope_pairing must be 'half' or 'adjacent', found {self.rope_pairing!r}")
        if self.rope_theta <= 0 or self.rms_norm_eps < 0:
            raise ConfigError("config.json: rope_theta must be positive and rms_norm_eps non-negative")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act {self.hidden_act!r} is not supported (silu only)")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError(
                    f"config.json: layer_types has {len(self.layer_types)} entries for "
                    f"{self.num_hidden_layers} layers")
            for t in self.layer_types:
                if t not in ("full_attention", "sliding_attention"):
                    raise ConfigError(f"config.json: unknown layer type {t!r}")
                if t == "sliding_attention" and self.sliding_window is None:
                    raise ConfigError("config.json: a sliding_attention layer needs sliding_window")

    # ---- writing -------------------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        d = {
            "architectures": [ARCHITECTURE],
            "model_type": "mistral",
            "num_hidden_layers": self.num_hidden_layers,
            "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "sliding_window": self.sliding_window,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": self.hidden_act,
            "torch_dtype": "bfloat16",
        }
        if self.rope_pairing != "half":
            d["rope_pairing"] = self.rope_pairing
        if self.layer_types is not None:
            d["layer_types"] = list(self.layer_types)
        if self.eos_token_id:
            d["eos_token_id"] = self.eos_token_id[0] if len(self.eos_token_id) == 1 else list(self.eos_token_id)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d

    def window_of_layer(self, i: int) -> Optional[int]:
        if self.sliding_window is None:
            return None
        if self.layer_types is None:
            return self.sliding_window
        return self.sliding_window if self.layer_types[i] == "sliding_attention" else None


def build_spec(cfg: MistralConfig) -> ModelSpec:
    """Mistral as parts: every layer is GQA attention + SwiGLU behind RMSNorms, pre-norm
    residual (reference: generic dense path, config.rs:497-510; layer loop
    megakernel/megakernel_compile.rs:115-236)."""
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layers: List[LayerSpec] = []
    for i in range(cfg.num_hidden_layers):
        mixer = PartSpec("gqa_attention", {
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "window": cfg.window_of_layer(i),
            "position": "rope",
            "scale": None,          # 1/sqrt(head_dim)
        })
        ffn = PartSpec("swiglu", {
            "hidden_size": cfg.hidden_size,
            "intermediate_size": cfg.intermediate_size,
        })
        # tensor names of MistralForCausalLM checkpoints (the reference looks the same ones up,
        # model_load.rs:624-744)
        layers.append(prenorm_layer(f"model.layers.{i}.", mixer, ffn, norm, norm, mixer_name="self_attn.",
                                    feed_forward_name="mlp.", mixer_norm_name="input_layernorm.",
                                    ffn_norm_name="post_attention_layernorm."))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        layers=layers,
        schedule=default_schedule(cfg.num_hidden_layers),
        final_norm=norm,
        lm_head=PartSpec("lm_head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                     "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None}),
        positions={"rope": PartSpec("rope", {"rotary_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                             "pairing": cfg.rope_pairing})},
        max_position_embeddings=cfg.max_position_embeddings,
        embedding_prefix="model.embed_tokens.", final_norm_prefix="model.norm.", lm_head_prefix="lm_head.",
        stop_token_ids=list(cfg.eos_token_id),
        bos_token_id=cfg.bos_token_id,
    )


# Shapes named by the benchmark description; usable without a model folder.
PRESETS: Dict[str, Dict[str, Any]] = {
    "tiny-a": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
                   head_dim=16, intermediate_size=192, vocab_size=256, rope_theta=10000.0,
                   rms_norm_eps=1e-5, sliding_window=None, max_position_embeddings=4096),
    "tiny-b": dict(num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3,
                   head_dim=32, intermediate_size=320, vocab_size=384, rope_theta=1e6,
                   rms_norm_eps=1e-6, sliding_window=8, max_position_embeddings=4096),
    "mistral-7b-v0.3": dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
                            num_key_value_heads=8, head_dim=128, intermediate_size=14336,
                            vocab_size=32768, rope_theta=1e6, rms_norm_eps=1e-5,
                            sliding_window=None, max_position_embeddings=32768),
    "mistral-7b-v0.1": dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32,
                            num_key_value_heads=8, head_dim=128, intermediate_size=14336,
                            vocab_size=32000, rope_theta=10000.0, rms_norm_eps=1e-5,
                            sliding_window=4096, max_position_embeddings=32768),
    "mistral-small-24b": dict(num_hidden_layers=40, hidden_size=5120, num_attention_heads=32,
                              num_key_value_heads=8, head_dim=128, intermediate_size=32768,
                              vocab_size=131072, rope_theta=1e8, rms_norm_eps=1e-5,
                              sliding_window=None, max_position_embeddings=32768),
}


def preset(name: str, **overrides) -> MistralConfig:
    if name not in PRESETS:
        raise ConfigError(f"unknown preset {name!r}; known: {sorted(PRESETS)}")
    d = dict(PRESETS[name])
    d.update(overrides)
    return MistralConfig.from_dict(d)
