from .step import StepBatch, Workspace, pack_step
from .model import DecoderModel, Layer
from .engine import Engine, StepEntry, parse_dtype
from .generate import generate, plan_batches, GenerationResult, GenerationStats

__all__ = ["StepBatch", "Workspace", "pack_step", "DecoderModel", "Layer", "Engine", "StepEntry", "parse_dtype", "generate", "plan_batches", "GenerationResult", "GenerationStats"]
