"""Named ranges around the phases of an iteration, for a profiler's timeline.

The switch is the reference's (src/cloud_engine/profiling.py:10-26): ranges are
emitted only when the environment has ``ENGINE_NVTX=1``.  It is read once, when
this module is imported; without it ``trace_range`` hands out one shared object
that does nothing, so a range costs a call and no more.  On ROCm torch's nvtx
functions emit roctx ranges, which ``rocprofv3 --marker-trace`` records.
"""

from __future__ import annotations

import os


class _NoRange:
    def __enter__(self) -> None:
        return None

    def __exit__(self, *exc: object) -> bool:
        return False


class _MarkedRange:
    __slots__ = ("name",)

    def __init__(self, name: str) -> None:
        self.name = name

    def __enter__(self) -> None:
        _push(self.name)

    def __exit__(self, *exc: object) -> bool:
        _pop()
        return False


def _markers():
    """torch's push and pop if ranges are wanted and torch can emit them, else nothing."""
    if os.environ.get("ENGINE_NVTX") != "1":
        return None
    try:
        import torch

        torch.cuda.nvtx.range_push("engine.ranges_on")
        torch.cuda.nvtx.range_pop()
    except (ImportError, RuntimeError):
        return None
    return torch.cuda.nvtx.range_push, torch.cuda.nvtx.range_pop


_ON = _markers()
_push, _pop = _ON if _ON is not None else (None, None)
_NOTHING = _NoRange()


def trace_range(name: str):
    """``with trace_range("phase"): ...``"""
    return _MarkedRange(name) if _ON is not None else _NOTHING
