"""MI355X-native inference engine for the Qwen2.5 dense decoder.

Import name ``cie_amd`` (see ``cie_amd.py`` at the repository root).

    from cie_amd import Engine, GenerationConfig
    engine = Engine("/path/to/model", dtype="bfloat16")
    results = engine.generate([[1, 2, 3]], GenerationConfig(max_output_tokens=8))
"""

__version__ = "0.1.0"

_LAZY = {
    "Engine": "engine", "GenerationConfig": "engine", "GenerationResult": "engine",
    "EngineConfig": "config", "build_engine_config": "config", "load_config": "config",
    "register_architecture": "config", "Qwen2Config": "config",
}


def __getattr__(name: str):
    if name in _LAZY:
        import importlib

        return getattr(importlib.import_module(f"{__name__}.{_LAZY[name]}"), name)
    raise AttributeError(name)
