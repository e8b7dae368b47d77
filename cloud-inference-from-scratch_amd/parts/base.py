"""Interfaces of the parts a decoder layer is put together from, and the
registries that map a :class:`~cie_amd.config.specs.PartSpec`'s ``kind`` to a
part class.

A part is built from its spec's parameters alone (sizes and constants; it never
learns which model it is in), says which checkpoint tensors it wants under a
name prefix, takes them in ``bind`` and then runs on the GPU.

Interfaces (``x`` is ``[tokens, hidden]`` in the engine's activation dtype,
``residual`` the float32 residual stream, ``batch`` a
:class:`~cie_amd.engine.batch.StepBatch`):

``Norm``        ``forward(residual, branch, out_dtype, rows=None) -> x``
                adds ``branch`` into ``residual`` (in place, float32) and returns
                the normalised rows.  A norm that sets ``takes_row_sumsq`` is
                also handed the ``RowSumsq`` / ``Added`` forms of a branch
                (``parts/linear.py``); any other gets a tensor or ``None``.
``Position``    ``tables(device) -> (cos, sin)`` or whatever its mixer asks of it.
``Mixer``       ``cache_need() -> PagedKV | FixedState | None`` and
                ``forward(x, batch, view, writes) -> y``; ``view`` is the cache
                unit of this call (``PagedView`` or ``StateView``), ``writes``
                tells whether this call appends to it.
``FeedForward`` ``forward(x) -> y``
``Block``       ``forward(residual, pending, batch, view, writes) -> (residual, pending)``
                ``pending`` is a branch output not yet added to the residual, so
                that the add fuses with the next norm.
"""

from __future__ import annotations

from typing import Any, Callable

import torch

from ..config.specs import PartSpec
from ..weights.tensors import TensorSpec

NORMS: dict[str, Callable[..., Any]] = {}
POSITIONS: dict[str, Callable[..., Any]] = {}
MIXERS: dict[str, Callable[..., Any]] = {}
FEED_FORWARDS: dict[str, Callable[..., Any]] = {}
BLOCKS: dict[str, Callable[..., Any]] = {}

_REGISTRIES = {
    "norm": NORMS,
    "position": POSITIONS,
    "mixer": MIXERS,
    "feed_forward": FEED_FORWARDS,
    "block": BLOCKS,
}


def register_part(role: str, kind: str, factory: Callable[..., Any]) -> None:
    """``role`` is one of norm, position, mixer, feed_forward, block."""
    _REGISTRIES[role][kind] = factory


def build_part(role: str, spec: PartSpec) -> Any:
    registry = _REGISTRIES[role]
    if spec.kind not in registry:
        raise KeyError(f"unknown {role} kind {spec.kind!r}; known: {sorted(registry)}")
    return registry[spec.kind](**spec.as_dict())


class Part:
    """Default behaviour of a part without tensors.

    ``graph_safe``: the part's ``forward`` reads everything that changes from
    step to step (lengths, slots, positions) from device tensors of the batch,
    never from its host lists, and launches the same kernels for the same batch
    size: only then may a decode step that contains it be captured in a graph."""

    graph_safe = False
    # ``adds_to_residual``: ``forward`` takes ``residual=`` and may add its output there itself
    # (returning a ``RowSumsq`` or an ``Added``).
    adds_to_residual = False

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        return {}

    def bind(self, tensors: dict[str, torch.Tensor], prefix: str, dtype: torch.dtype,
             device: torch.device) -> None:
        self.dtype = dtype
        self.device = device
