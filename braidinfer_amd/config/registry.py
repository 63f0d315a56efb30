"""One registry from an architecture's name to its configuration class and builder.

The reference has no registry: it sniffs keys (`layer_types`, `num_experts`, ...) and
tests `model_type` strings (crates/braidinfer-runtime/src/config.rs:357-369,406-510).
Here the key is ``config.json["architectures"][0]``, with `model_type` as a second
name for folders that omit `architectures`.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional

from ..errors import ConfigError
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any                      # has from_dict(dict) and to_dict()
    build_spec: Callable[[Any], ModelSpec]
    model_type: Optional[str] = None


_ARCHITECTURES: Dict[str, Architecture] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_class, build_spec, model_type: Optional[str] = None,
                          replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ConfigError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec, model_type)
    if model_type is not None:
        _MODEL_TYPES[model_type] = name


def unregister_architecture(name: str) -> None:
    arch = _ARCHITECTURES.pop(name, None)
    if arch is not None and arch.model_type is not None:
        _MODEL_TYPES.pop(arch.model_type, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def architecture_of(config_dict: Dict[str, Any]) -> Architecture:
    archs = config_dict.get("architectures")
    name = None
    if isinstance(archs, (list, tuple)) and archs:
        name = archs[0]
    elif isinstance(archs, str):
        name = archs
    if name is None:
        mt = config_dict.get("model_type")
        if mt in _MODEL_TYPES:
            name = _MODEL_TYPES[mt]
        else:
            raise ConfigError(
                "config.json names no architecture ('architectures' is absent and model_type "
                f"{mt!r} is unknown); registered: {registered_architectures()}")
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def architecture_of_config(config) -> Architecture:
    name = getattr(config, "architecture", None)
    if name not in _ARCHITECTURES:
        raise ConfigError(f"configuration {type(config).__name__} names unknown architecture {name!r}; "
                          f"registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder}: no config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return d


def generation_stop_tokens(folder: str):
    """`eos_token_id` (an integer or a list) of the folder's generation_config.json, [] when
    the file or the key is absent.  The reference gathers its stop set from the tokenizer's
    end markers and config.json's `text_config.eos_token_id`
    (crates/braidinfer-runtime/src/generate.rs:34-68); checkpoints of this architecture
    carry theirs in config.json and in generation_config.json, and both are read."""
    path = os.path.join(folder, "generation_config.json")
    if not os.path.isfile(path):
        return []
    try:
        with open(path, "r", encoding="utf-8") as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    eos = d.get("eos_token_id") if isinstance(d, dict) else None
    if eos is None:
        return []
    ids = [eos] if isinstance(eos, int) and not isinstance(eos, bool) else eos
    if not isinstance(ids, (list, tuple)) or not all(isinstance(e, int) and not isinstance(e, bool) and e >= 0 for e in ids):
        raise ConfigError(f"{path}: eos_token_id must be a token id or a list of them, found {eos!r}")
    return list(ids)


def config_from_dict(d: Dict[str, Any]):
    arch = architecture_of(d)
    return arch.config_class.from_dict(d)


def config_from_folder(folder: str):
    return config_from_dict(read_config_json(folder))


def spec_of(config) -> ModelSpec:
    return architecture_of_config(config).build_spec(config)
