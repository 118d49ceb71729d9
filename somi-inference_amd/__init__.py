"""An MI355X-native inference engine for the Qwen2.5 dense decoder.

Everything between a request's tokens and its next token on one GPU: typed
configuration and an architecture registry, weights from safetensors by name,
layers put together from parts, a paged cache manager, one step function for
mixed batches, a scheduler, sampling, and hand-written HIP kernels for gfx950.
"""

from . import config as config
from . import models as _models            # registers the architectures  # noqa: F401
from .config import ConfigError, EngineConfig, Qwen2Config
from .entrypoints import LLM
from .sampling import SamplingParams

__version__ = "0.1.0"
__all__ = ["ConfigError", "EngineConfig", "LLM", "Qwen2Config", "SamplingParams", "config"]
