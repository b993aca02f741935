"""synaptix_amd: a small Qwen3 dense decoder library with generation of its own for one MI355X."""
from .config import ConfigError, Qwen3Config, load_config, register_architecture, known_architectures
from .weights import WeightError, write_random_model
from .cache import CacheFull, CacheError
from . import models as _models  # registers the architectures
from .engine import Engine, StepError
from .engine.generate import generate, GenerationOutput, GenerationStats
from .sampling import GenerationConfig
from .pipeline import Pipeline, load

__all__ = ["ConfigError", "Qwen3Config", "load_config", "register_architecture", "known_architectures",
           "WeightError", "write_random_model", "CacheFull", "CacheError", "Engine", "StepError", "generate",
           "GenerationOutput", "GenerationStats", "GenerationConfig", "Pipeline", "load"]
__version__ = "0.1.0"
