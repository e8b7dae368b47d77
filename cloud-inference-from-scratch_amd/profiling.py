"""Optional trace ranges around scheduler and step phases.

Same switch as the reference's ``nvtx_range`` (src/cloud_engine/profiling.py:10-26):
nothing happens unless ``ENGINE_NVTX=1``.  On ROCm torch's nvtx calls emit roctx
ranges, which rocprofv3 records with ``--marker-trace``.
"""

from __future__ import annotations

import contextlib
import os
from collections.abc import Iterator


@contextlib.contextmanager
def trace_range(name: str) -> Iterator[None]:
    if os.environ.get("ENGINE_NVTX") != "1":
        yield
        return
    try:
        import torch

        torch.cuda.nvtx.range_push(name)
    except (ImportError, RuntimeError):
        yield
        return
    try:
        yield
    finally:
        with contextlib.suppress(RuntimeError):
            torch.cuda.nvtx.range_pop()
