"""braidinfer_amd: a small generation library for one MI355X (gfx950).

From a model folder (config.json + safetensors) or a configuration and a seed to
generated tokens: typed configuration and architecture registry, weights by tensor
name, layers put together from parts, a paged cache with a slot per sequence, one
batched step function, a generation loop with the reference's sampler, and trace
replay.  Every device operation is a hand-written HIP kernel under `csrc/`.
"""
from .errors import BraidError, ConfigError, WeightError, CacheError, KernelError, StepError
from .config import (MistralConfig, preset, PRESETS, config_from_folder, config_from_dict, spec_of,
                     register_architecture, registered_architectures, PartSpec, LayerSpec, ScheduleEntry,
                     ModelSpec, prenorm_layer)
from .parts import register_part
from .engine import Engine, StepEntry, DecoderModel, generate, GenerationResult, GenerationStats
from .sampling import SamplingParams, Sampler

__version__ = "0.1.0"

__all__ = ["BraidError", "ConfigError", "WeightError", "CacheError", "KernelError", "StepError",
           "MistralConfig", "preset", "PRESETS", "config_from_folder", "config_from_dict", "spec_of",
           "register_architecture", "registered_architectures", "PartSpec", "LayerSpec", "ScheduleEntry",
           "ModelSpec", "prenorm_layer", "register_part", "Engine", "StepEntry", "DecoderModel", "generate", "GenerationResult",
           "GenerationStats", "SamplingParams", "Sampler"]
