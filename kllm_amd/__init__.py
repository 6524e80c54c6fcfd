"""kllm_amd: a small inference engine for AMD MI355X (gfx950).

Everything between a request's token ids and its next token: typed
configuration and a registry of architectures, weights by tensor name, layers
put together from parts, a paged cache manager, one step function over mixed
batches, a continuous-batching scheduler, greedy and temperature sampling, and
hand-written HIP kernels for prompts and for decoding.
"""

from . import models  # registers the built-in architecture
from .cache import CacheManager, OutOfPages
from .config import ConfigError, LlamaConfig, load_config, register_architecture
from .engine import Engine, EngineOptions, Scheduler, StepEntry
from .parts import PartSpec, register_part
from .weights import WeightError, write_random_model

__version__ = "0.1.0"
__all__ = ["CacheManager", "OutOfPages", "ConfigError", "LlamaConfig", "load_config",
           "register_architecture", "Engine", "EngineOptions", "Scheduler", "StepEntry",
           "PartSpec", "register_part", "WeightError", "write_random_model"]
