from .engine_config import EngineConfig
from .registry import (ConfigError, build_spec, config_class, config_from_dict, known_architectures,
                       load_config, register_architecture)
from .spec import LayerSpec, ModelSpec, PartSpec, Run, layer
from .qwen2 import Qwen2Config
from .presets import PRESETS, preset

__all__ = ["EngineConfig", "ConfigError", "build_spec", "config_class", "config_from_dict",
           "known_architectures", "load_config", "register_architecture", "LayerSpec", "ModelSpec",
           "PartSpec", "Run", "layer", "Qwen2Config", "PRESETS", "preset"]
