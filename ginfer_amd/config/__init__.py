from .registry import (ConfigError, register_architecture, registered_architectures, config_class,
                       config_from_dict, config_from_folder)
from .spec import PartSpec, LayerSpec, prenorm_layer, ScheduleEntry, ModelSpec
from .qwen2 import Qwen2Config

__all__ = ["ConfigError", "register_architecture", "registered_architectures", "config_class",
           "config_from_dict", "config_from_folder", "PartSpec", "LayerSpec", "prenorm_layer", "ScheduleEntry",
           "ModelSpec", "Qwen2Config"]
