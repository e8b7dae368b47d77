"""The one registry from an architecture's name (``config.json``'s
``architectures[0]``) to its typed configuration and model builder.

The reference has no registry, only a ``model_type`` set check
(src/cloud_engine/model.py:61-63).  Here a new architecture is one call to
:func:`register_architecture`; the default builder assembles the generic
decoder from the configuration's :class:`~cie_amd.config.specs.ModelSpec`.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

from .specs import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Any
    build_model: Callable[..., Any] | None = None  # None: the generic decoder from model_spec()


ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_TYPES: dict[str, str] = {}


def register_architecture(
    name: str,
    config_class: Any,
    build_model: Callable[..., Any] | None = None,
    model_type: str | None = None,
) -> None:
    """Make ``name`` loadable.  ``config_class`` needs ``from_hf_config(dict)``,
    ``to_hf_config()`` and ``model_spec()``."""
    ARCHITECTURES[name] = Architecture(name, config_class, build_model)
    if model_type is not None:
        _MODEL_TYPES[model_type] = name


def architecture_of(raw: dict[str, Any]) -> Architecture:
    names = raw.get("architectures") or []
    name = names[0] if names else _MODEL_TYPES.get(raw.get("model_type", ""))
    if name is None or name not in ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name or raw.get('model_type')!r}; known: {sorted(ARCHITECTURES)}"
        )
    return ARCHITECTURES[name]


def config_from_dict(raw: dict[str, Any]) -> Any:
    return architecture_of(raw).config_class.from_hf_config(raw)


def load_config(model_dir: str | Path) -> Any:
    """Read ``config.json`` of a model folder into its architecture's typed configuration."""
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in {model_dir}")
    with open(path, encoding="utf-8") as handle:
        return config_from_dict(json.load(handle))

