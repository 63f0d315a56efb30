from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec, default_schedule, prenorm_layer
from .registry import (Architecture, register_architecture, unregister_architecture,
                       registered_architectures, architecture_of, architecture_of_config,
                       read_config_json, config_from_dict, config_from_folder, spec_of, generation_stop_tokens)
from .mistral import MistralConfig, PRESETS, preset, build_spec as build_mistral_spec, ARCHITECTURE as MISTRAL

register_architecture(MISTRAL, MistralConfig, build_mistral_spec, model_type="mistral", replace=True)

__all__ = [
    "PartSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "default_schedule", "prenorm_layer",
    "Architecture", "register_architecture", "unregister_architecture", "registered_architectures",
    "architecture_of", "architecture_of_config", "read_config_json", "config_from_dict",
    "config_from_folder", "spec_of", "generation_stop_tokens", "MistralConfig", "PRESETS", "preset",
]
