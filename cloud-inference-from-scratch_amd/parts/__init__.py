from . import attention, block, feed_forward, norm, position  # noqa: F401  (fill the registries)
from .base import (
    BLOCKS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITIONS,
    Part,
    build_part,
    register_part,
)
from .model import DecoderModel, expected_tensors

__all__ = [
    "BLOCKS", "DecoderModel", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "Part",
    "build_part", "expected_tensors", "register_part",
]
