from .spec import (ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry,
                   default_schedule)
from .lfm2 import Lfm2Config
from .registry import (architecture_name, config_from_dict, load_config,
                       register_architecture, registered_architectures)

register_architecture("Lfm2ForCausalLM", Lfm2Config)
register_architecture("lfm2", Lfm2Config)

__all__ = [
    "ConfigError", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry", "default_schedule",
    "Lfm2Config", "architecture_name", "config_from_dict", "load_config",
    "register_architecture", "registered_architectures",
]
