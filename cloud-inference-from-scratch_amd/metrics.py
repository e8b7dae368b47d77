"""What the engine counts while it serves: totals since the last reset, and the
latest latencies in windows of bounded length.

The figures are those of the reference's ``Metrics``
(src/cloud_engine/metrics.py:52-200): time to the first token, time between
tokens and whole-request time with their percentiles; requests by outcome;
tokens taken in, produced and computed twice; the size of each iteration's
batch.  The scheduler writes into :class:`Totals` and the :class:`Window`
objects directly.
"""

from __future__ import annotations

import math
from collections import deque
from collections.abc import Iterable
from dataclasses import asdict, dataclass
from typing import Any


def quantile(samples: Iterable[float], fraction: float) -> float:
    """The value at ``fraction`` (0..1) of the way through the sorted samples,
    weighted between the two neighbours it falls between; 0 for no samples."""
    ranked = sorted(samples)
    if not ranked:
        return 0.0
    place = min(max(fraction, 0.0), 1.0) * (len(ranked) - 1)
    under = math.floor(place)
    weight = place - under
    if weight == 0.0:
        return ranked[under]
    return (1.0 - weight) * ranked[under] + weight * ranked[under + 1]


class Window:
    """The latest ``length`` samples of one latency."""

    def __init__(self, length: int) -> None:
        self._samples: deque[float] = deque(maxlen=length)

    def add(self, value: float) -> None:
        self._samples.append(value)

    def __len__(self) -> int:
        return len(self._samples)

    def summary(self) -> dict[str, float]:
        out: dict[str, float] = {"count": len(self._samples)}
        for name, fraction in (("p50", 0.50), ("p95", 0.95), ("p99", 0.99)):
            out[name] = quantile(self._samples, fraction)
        return out


@dataclass
class Totals:
    completed: int = 0
    failed: int = 0
    cancelled: int = 0
    rejected: int = 0
    preempted: int = 0
    iterations: int = 0
    input_tokens: int = 0
    output_tokens: int = 0
    recomputed_tokens: int = 0


class Metrics:
    def __init__(self, latency_samples: int = 4096, batch_samples: int = 16_384) -> None:
        self._lengths = (latency_samples, batch_samples)
        self.reset()

    def reset(self) -> None:
        """Start counting afresh (after a warm-up, before a measured run)."""
        latency_samples, batch_samples = self._lengths
        self.totals = Totals()
        self.first_token_ms = Window(latency_samples)
        self.between_tokens_ms = Window(latency_samples)
        self.whole_request_ms = Window(latency_samples)
        self.batch_sizes: deque[int] = deque(maxlen=batch_samples)

    def iteration(self, requests: int, tokens: int) -> None:
        self.totals.iterations += 1
        self.totals.input_tokens += tokens
        self.batch_sizes.append(requests)

    def snapshot(self) -> dict[str, Any]:
        totals = asdict(self.totals)
        sizes = self.batch_sizes
        return {
            "latency_ms": {"ttft": self.first_token_ms.summary(), "itl": self.between_tokens_ms.summary(),
                           "e2e": self.whole_request_ms.summary()},
            "requests": {f"{outcome}_total": totals[outcome]
                         for outcome in ("completed", "failed", "cancelled", "rejected", "preempted")},
            "tokens": {"input_total": totals["input_tokens"], "output_total": totals["output_tokens"],
                       "recomputed_total": totals["recomputed_tokens"]},
            "scheduler": {"iterations_total": totals["iterations"],
                          "mean_batch_size": sum(sizes) / len(sizes) if sizes else 0.0,
                          "max_batch_size": max(sizes, default=0)},
        }
