"""flyweight_amd: a small, whole LFM2 inference engine for the AMD Instinct MI355X."""

from .config import ConfigError, Lfm2Config, load_config, register_architecture, registered_architectures
from .engine import EngineError, Model, Runtime, StepEntry
from .sampling import SamplingConfig

__version__ = "0.1.0"

__all__ = ["ConfigError", "Lfm2Config", "load_config", "register_architecture", "registered_architectures",
           "EngineError", "Model", "Runtime", "StepEntry", "SamplingConfig", "__version__"]
