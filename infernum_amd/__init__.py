"""infernum_amd: a small, whole inference engine for one MI355X (gfx950)."""
from . import parts as _parts          # noqa: F401  registers the built-in parts
from . import models as _models        # noqa: F401  registers the built-in architectures
from .cache import CacheConfig
from .config import ConfigError, LlamaConfig, UnsupportedModelError, load_config, register_architecture
from .engine import (BatchConfig, Engine, FinishReason, GenerationError, GenerationEvent, OutOfPages, Runtime,
                     Scheduler, StepEntry)
from .sampling import GenerateOptions, SamplingParams
from .parts import register_part

__version__ = "0.1.0"
