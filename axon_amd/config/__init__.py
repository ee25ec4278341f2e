from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, read_config_json)
from .engine import EngineConfig, dtype_name
from .registry import (architecture_of, config_from_dict, config_from_dir, known_architectures,
                       register_architecture)
from .qwen2 import Qwen2Config

__all__ = ["ConfigError", "LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "Run", "read_config_json",
           "EngineConfig", "dtype_name", "architecture_of", "config_from_dict", "config_from_dir",
           "known_architectures", "register_architecture", "Qwen2Config"]

register_architecture(Qwen2Config.architecture, Qwen2Config, Qwen2Config.model_type)
