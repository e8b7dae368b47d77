from .engine_config import EngineConfig, build_engine_config, canonical_dtype
from .qwen2 import Qwen2Config
from .registry import (
    ARCHITECTURES,
    Architecture,
    architecture_of,
    config_from_dict,
    load_config,
    register_architecture,
)
from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

# the architectures this package brings; others register themselves the same way from outside
register_architecture("Qwen2ForCausalLM", Qwen2Config, model_type="qwen2")

__all__ = [
    "ARCHITECTURES", "Architecture", "ConfigError", "EngineConfig", "LayerCall", "LayerSpec",
    "ModelSpec", "PartSpec", "Qwen2Config", "architecture_of", "build_engine_config",
    "canonical_dtype", "config_from_dict", "load_config", "register_architecture",
]
