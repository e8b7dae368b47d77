"""What a part says about each tensor it wants from a checkpoint."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class TensorSpec:
    """``shape`` as stored.  ``init`` tells the random-weights mode how to fill
    it: ``"normal"`` is N(0, std), ``"norm"`` is 1 + N(0, std).  ``kind`` is
    ``"float"`` (runs in the engine's dtype) or ``"int"`` (kept as int32).
    ``keeps_float32``: a small vector (norm weight) that stays in 32-bit when the
    file stores it so, whatever the engine's dtype."""

    shape: tuple[int, ...]
    init: str = "normal"
    kind: str = "float"
    keeps_float32: bool = False
