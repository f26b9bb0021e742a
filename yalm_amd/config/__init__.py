from .llama import ConfigError, LlamaConfig, RopeScaling
from .registry import (config_from_dict, config_from_folder, register_architecture, registered_architectures,
                       unregister_architecture)
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = ["ConfigError", "LlamaConfig", "RopeScaling", "config_from_dict", "config_from_folder",
           "register_architecture", "registered_architectures", "unregister_architecture", "LayerSpec", "ModelSpec",
           "PartSpec", "ScheduleEntry"]
