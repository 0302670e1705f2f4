from .base import KeyReader, LayerSpec, ModelConfig, PartSpec, ScheduleEntry, read_config_json
from .qwen2 import Qwen2Config
from .registry import (
    architecture_names,
    architecture_of,
    config_from_dict,
    load_config,
    lookup_architecture,
    register_architecture,
    unregister_architecture,
)

__all__ = [
    "KeyReader", "LayerSpec", "ModelConfig", "PartSpec", "ScheduleEntry", "read_config_json",
    "Qwen2Config", "architecture_names", "architecture_of", "config_from_dict", "load_config",
    "lookup_architecture", "register_architecture", "unregister_architecture",
]
