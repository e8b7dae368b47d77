from .engine_config import EngineConfig, build_engine_config, canonical_dtype
from .qwen2 import ConfigError, Qwen2Config
from .registry import (
    ARCHITECTURES,
    Architecture,
    architecture_of,
    config_from_dict,
    load_config,
    register_architecture,
)
from .specs import LayerCall, LayerSpec, ModelSpec, PartSpec

__all__ = [
    "ARCHITECTURES", "Architecture", "ConfigError", "EngineConfig", "LayerCall", "LayerSpec",
    "ModelSpec", "PartSpec", "Qwen2Config", "architecture_of", "build_engine_config",
    "canonical_dtype", "config_from_dict", "load_config", "register_architecture",
]
