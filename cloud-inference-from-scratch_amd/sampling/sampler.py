"""Greedy and temperature sampling over a step's float32 logits.

The reference samples greedily only: ``argmax(logits.float())``
(src/cloud_engine/engine.py:486-487, src/cloud_engine/model.py:231-233) and
refuses any other temperature (src/cloud_engine/scheduler.py:69-71).  Here
``temperature > 0`` draws from ``softmax(logits / temperature)`` by inverse CDF
with one uniform number per row.  That number is a hash of (seed, the request's
serial number unless it brought its own seed, index of the generated token): a
request's draws are the same whatever else is in the batch, however its prompt
was cut, and after a preemption.
"""

from __future__ import annotations

from collections.abc import Sequence

import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def _mix(value: int) -> int:
    """splitmix64 finaliser."""
    value = (value + 0x9E3779B97F4A7C15) & _MASK
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK
    return value ^ (value >> 31)


def uniform_for(seed: int, stream: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in float32)."""
    word = _mix(_mix(_mix(seed & _MASK) ^ (stream & _MASK)) ^ (index & _MASK))
    return (word >> 40) / float(1 << 24)


class Sampler:
    def __init__(self, seed: int = 0) -> None:
        self.seed = seed

    def uniform(self, request_seed: int | None, serial: int, index: int) -> float:
        if request_seed is not None:
            return uniform_for(request_seed, 0, index)
        return uniform_for(self.seed, serial, index)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float],
               uniforms: Sequence[float]) -> list[int]:
        """One token per row of ``logits`` [n, vocab] (float32, on the GPU)."""
        if logits.shape[0] == 0:
            return []
        return self.sample_on_device(logits, temperatures, uniforms).tolist()

    def sample_on_device(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: Sequence[float],
                         out: torch.Tensor | None = None) -> torch.Tensor:
        """The same, left on the GPU (int32 [n], in ``out`` if given): nothing waits for the result."""
        if all(t == 0 for t in temperatures):
            return ops.sample(logits, out=out)
        # one page-locked block for both, copied without waiting: the decode steps that are started ahead of
        # their tokens must not stop the host here (a copy from pageable memory would)
        rows = len(temperatures)
        pinned = logits.device.type == "cuda"
        staged = torch.tensor([*temperatures, *uniforms], dtype=torch.float32, pin_memory=pinned)
        on_device = staged.to(logits.device, non_blocking=True)
        return ops.sample(logits, on_device[:rows], on_device[rows:], out=out)
