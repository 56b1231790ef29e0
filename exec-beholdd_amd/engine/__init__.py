"""The step function, the engine around it and the generation loop above it."""

from .engine import Engine, load_model, parse_dtype, random_model_on_device
from .generation import (FINISH_LENGTH, FINISH_STOP, GenerationError, GenerationResult, generate,
                         plan_batches, positions_needed)
from .step import StepEntry, StepError, build_step
from . import artifact, replay

__all__ = ["Engine", "load_model", "parse_dtype", "random_model_on_device", "FINISH_LENGTH", "FINISH_STOP",
           "GenerationError", "GenerationResult", "generate", "plan_batches", "positions_needed",
           "StepEntry", "StepError", "build_step"]
