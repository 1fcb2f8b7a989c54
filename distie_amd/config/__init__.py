from .engine_config import EngineConfig, resolve_dtype
from .model_config import (ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec, Qwen2Config,
                           read_config_json)
from .registry import (architecture_of, config_from_dict, known_architectures, load_model_config,
                       model_spec_from_dir, register_architecture)

__all__ = [
    "EngineConfig", "resolve_dtype", "ConfigError", "LayerCall", "LayerSpec", "ModelSpec", "PartSpec",
    "Qwen2Config", "read_config_json", "architecture_of", "config_from_dict", "known_architectures",
    "load_model_config", "model_spec_from_dir", "register_architecture",
]
