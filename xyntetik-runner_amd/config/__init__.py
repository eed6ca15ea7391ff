from .base import ConfigError, Fields, read_config_json, architecture_name
from .llama import LlamaConfig, RopeScaling
from .spec import PartSpec, LayerSpec, ExecStep, ModelSpec
from .registry import (register_architecture, unregister_architecture, get_architecture,
                       known_architectures, load_config, config_from_dict, Architecture)

__all__ = [
    "ConfigError", "Fields", "read_config_json", "architecture_name", "LlamaConfig", "RopeScaling",
    "PartSpec", "LayerSpec", "ExecStep", "ModelSpec", "register_architecture",
    "unregister_architecture", "get_architecture", "known_architectures", "load_config",
    "config_from_dict", "Architecture",
]
