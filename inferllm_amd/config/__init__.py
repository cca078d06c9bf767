from .registry import (ConfigError, config_class, config_from_dict, load_config,
                       register_architecture, registered_architectures)
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = ["ConfigError", "config_class", "config_from_dict", "load_config",
           "register_architecture", "registered_architectures",
           "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry"]
