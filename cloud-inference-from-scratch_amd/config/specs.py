"""Architecture-neutral descriptions of a decoder: what an architecture's
configuration is turned into before any tensor exists.

A model is a list of layers, each a :class:`LayerSpec` that names its mixer,
feed-forward, norms and arrangement by *kind* (a key of the part registries in
``cie_amd.parts``) together with every size and constant the part needs, and an
*order*: the list of :class:`LayerCall` that says which layer runs when and on
which cache.  Nothing here knows a model family; a configuration class (for
instance ``Qwen2Config``) produces these from its own ``config.json`` keys.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


class ConfigError(ValueError):
    """A ``config.json`` that no registered architecture can run: an unknown name, a key
    that is missing, a value outside what the parts take."""


@dataclass(frozen=True)
class PartSpec:
    """``kind`` selects the part class; ``params`` are its constructor arguments."""

    kind: str
    params: tuple[tuple[str, Any], ...] = ()

    @classmethod
    def of(cls, kind: str, **params: Any) -> "PartSpec":
        return cls(kind, tuple(sorted(params.items())))

    def as_dict(self) -> dict[str, Any]:
        return dict(self.params)


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which parts, how arranged, and under which tensor names.

    ``names`` maps the block's part roles (``norm1``, ``mixer``, ``norm2``,
    ``feed_forward``) to the sub-prefix of the checkpoint's tensor names.
    """

    mixer: PartSpec
    feed_forward: PartSpec
    norm1: PartSpec
    norm2: PartSpec
    block: str = "pre_norm"
    names: tuple[tuple[str, str], ...] = ()

    def name_of(self, role: str) -> str:
        return dict(self.names).get(role, role)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer``  index into ``ModelSpec.layers`` (a layer may be named twice).
    ``cache``  index of the cache unit the mixer reads; two calls may name the
               same unit, then the later one reads what the earlier one wrote.
    ``writes`` whether this call appends its own keys/values (or state) to the
               unit before reading it.
    """

    layer: int
    cache: int
    writes: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerSpec, ...]
    order: tuple[LayerCall, ...]
    final_norm: PartSpec
    tie_word_embeddings: bool
    max_position: int
    eos_token_id: int | None = None
    embedding_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head.weight"
    layer_prefix: str = "model.layers.{index}."
    extra: dict[str, Any] = field(default_factory=dict, compare=False)

    def __post_init__(self) -> None:
        units: dict[int, int] = {}
        for call in self.order:
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order names layer {call.layer}, model has {len(self.layers)}")
            if call.cache < 0:
                raise ValueError("cache unit indices are non-negative")
            if call.writes:
                units.setdefault(call.cache, call.layer)
        for call in self.order:
            if call.cache not in units:
                raise ValueError(f"cache unit {call.cache} is read by layer {call.layer} but never written")

    @property
    def cache_units(self) -> int:
        return max((call.cache for call in self.order), default=-1) + 1
