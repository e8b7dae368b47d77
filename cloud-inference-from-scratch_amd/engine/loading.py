"""From a model folder (or a configuration and a seed) to a model on the GPU."""

from __future__ import annotations

from pathlib import Path
from typing import Any

import torch

from ..config.engine_config import canonical_dtype
from ..config.registry import ARCHITECTURES, load_config
from ..parts.model import DecoderModel
from ..weights.loader import RandomSource, SafetensorsSource


def build_model(config: Any) -> DecoderModel:
    """The model object of a typed configuration, chosen by its architecture's registry entry."""
    entry = ARCHITECTURES.get(getattr(config, "architecture", None))
    if entry is None:
        raise KeyError(f"configuration {type(config).__name__} belongs to no registered architecture")
    if entry.build_model is not None:
        return entry.build_model(config)
    return DecoderModel(config.model_spec())


def load_model(model_dir: str | Path, dtype: str = "bfloat16",
               device: str | torch.device = "cuda:0") -> tuple[DecoderModel, Any]:
    """Read ``config.json`` and every ``*.safetensors`` of ``model_dir``."""
    config = load_config(model_dir)
    model = build_model(config)
    model.load(SafetensorsSource(model_dir), canonical_dtype(dtype), device)
    return model, config


def random_model(config: Any, seed: int, dtype: str = "bfloat16", device: str | torch.device = "cuda:0",
                 draw_device: str = "cpu") -> DecoderModel:
    """Random-weights mode without a folder: the same tensors ``write_model_folder`` would store."""
    model = build_model(config)
    model.load(RandomSource(seed, draw_device=draw_device), canonical_dtype(dtype), device)
    return model
