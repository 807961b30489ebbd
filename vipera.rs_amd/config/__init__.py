from .base import KeyReader, LayerSpec, ModelConfig, PartSpec, ScheduleEntry, read_config_json
from .gilidra import GilidraConfig
from .lurirax import LuriraxConfig
from .muzasun import MuzasunConfig
from .qwen2 import Qwen2Config
from .zulesun import ZulesunConfig
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
    "GilidraConfig", "LuriraxConfig", "MuzasunConfig", "Qwen2Config", "ZulesunConfig", "architecture_names", "architecture_of", "config_from_dict", "load_config",
    "lookup_architecture", "register_architecture", "unregister_architecture",
]
