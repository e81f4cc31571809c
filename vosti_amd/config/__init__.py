from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .registry import (ConfigError, architecture_names, config_from_dict, load_config, register_architecture,
                       resolve_architecture)
from .qwen3 import Qwen3Config

__all__ = ["LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry", "ConfigError", "architecture_names",
           "config_from_dict", "load_config", "register_architecture", "resolve_architecture", "Qwen3Config"]
