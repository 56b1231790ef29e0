"""The step function, the engine around it and the generation loop above it."""

from .engine import Engine, MemoryBudgetError, load_model, open_model, parse_dtype, random_model_on_device
from .generation import (FINISH_LENGTH, FINISH_STOP, GenerationError, GenerationResult, decode_ahead, generate,
                         plan_batches, positions_needed)
from .step import StepEntry, StepError, StepLayout, build_step, cache_for_runs
from . import artifact, compare, replay

__all__ = ["Engine", "MemoryBudgetError", "open_model", "StepLayout", "cache_for_runs", "load_model", "parse_dtype", "random_model_on_device", "FINISH_LENGTH", "FINISH_STOP",
           "GenerationError", "GenerationResult", "decode_ahead", "generate", "plan_batches", "positions_needed",
           "StepEntry", "StepError", "build_step"]
