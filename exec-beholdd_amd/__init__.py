"""beholdd for MI355X: a small model library with generation of its own.

One architecture (Qwen3 dense), one GPU, everything between a request's token ids and its
next token: typed configuration and registry, safetensors weights, parts assembled into a
decoder, a paged per-sequence cache, one step function, a generation loop with sampling, and
hand-written gfx950 kernels underneath.

The folder's name is not a Python identifier; import it with
`importlib.import_module("exec-beholdd_amd")` or through the `beholdd` module beside it.
"""

from . import config, weights, parts, cache, kernels, sampling, registry, models, engine, cli   # noqa: F401
from .config import ConfigError, ConfigReader, LayerKinds, Qwen3Config
from .engine import Engine, GenerationResult, MemoryBudgetError, StepEntry, load_model
from .registry import register_architecture, registered_architectures, resolve_architecture
from .sampling import SamplingParams
from .weights import WeightError, write_random_model

__version__ = "0.1.0"

__all__ = ["ConfigError", "ConfigReader", "LayerKinds", "MemoryBudgetError", "Qwen3Config", "Engine", "GenerationResult", "StepEntry", "load_model",
           "register_architecture", "registered_architectures", "resolve_architecture", "SamplingParams",
           "WeightError", "write_random_model"]
