"""Bounded counters and latency windows, after the reference's ``Metrics``
(src/cloud_engine/metrics.py:52-200): TTFT / ITL / E2E samples in fixed-capacity
windows, totals for requests and tokens, batch sizes per iteration."""

from __future__ import annotations

from collections import deque
from typing import Any


def percentile(values: list[float], pct: float) -> float:
    """Linear interpolation on a sorted copy; empty input gives 0 (metrics.py:19-31)."""
    if not values:
        return 0.0
    ordered = sorted(values)
    if len(ordered) == 1:
        return ordered[0]
    rank = (len(ordered) - 1) * (pct / 100.0)
    lower = int(rank)
    upper = min(lower + 1, len(ordered) - 1)
    return ordered[lower] + (ordered[upper] - ordered[lower]) * (rank - lower)


class Metrics:
    def __init__(self, latency_capacity: int = 4096) -> None:
        self._latency_capacity = latency_capacity
        self.reset()

    def reset(self) -> None:
        """Forget everything recorded so far (after a warm-up, before a measured run)."""
        latency_capacity = self._latency_capacity
        self._ttft: deque[float] = deque(maxlen=latency_capacity)
        self._itl: deque[float] = deque(maxlen=latency_capacity)
        self._e2e: deque[float] = deque(maxlen=latency_capacity)
        self._batch_sizes: deque[int] = deque(maxlen=16_384)
        self.completed_total = 0
        self.failed_total = 0
        self.cancelled_total = 0
        self.rejected_total = 0
        self.preempted_total = 0
        self.iterations_total = 0
        self.input_tokens_total = 0
        self.output_tokens_total = 0
        self.recomputed_tokens_total = 0

    def record_ttft_ms(self, value: float) -> None:
        self._ttft.append(value)

    def record_itl_ms(self, value: float) -> None:
        self._itl.append(value)

    def record_e2e_ms(self, value: float) -> None:
        self._e2e.append(value)

    def record_iteration(self, batch_size: int) -> None:
        self.iterations_total += 1
        self._batch_sizes.append(batch_size)

    def record_input_tokens(self, count: int) -> None:
        self.input_tokens_total += count

    def record_output_token(self, count: int = 1) -> None:
        self.output_tokens_total += count

    def record_recomputed_tokens(self, count: int) -> None:
        self.recomputed_tokens_total += count

    def inc_completed(self) -> None:
        self.completed_total += 1

    def inc_failed(self) -> None:
        self.failed_total += 1

    def inc_cancelled(self) -> None:
        self.cancelled_total += 1

    def inc_rejected(self) -> None:
        self.rejected_total += 1

    def inc_preempted(self) -> None:
        self.preempted_total += 1

    @staticmethod
    def _summary(samples: deque) -> dict[str, float]:
        values = list(samples)
        return {"count": len(values), "p50": percentile(values, 50), "p95": percentile(values, 95),
                "p99": percentile(values, 99)}

    def snapshot(self) -> dict[str, Any]:
        sizes = list(self._batch_sizes)
        return {
            "latency_ms": {"ttft": self._summary(self._ttft), "itl": self._summary(self._itl),
                           "e2e": self._summary(self._e2e)},
            "requests": {
                "completed_total": self.completed_total, "failed_total": self.failed_total,
                "cancelled_total": self.cancelled_total, "rejected_total": self.rejected_total,
                "preempted_total": self.preempted_total,
            },
            "tokens": {
                "input_total": self.input_tokens_total, "output_total": self.output_tokens_total,
                "recomputed_total": self.recomputed_tokens_total,
            },
            "scheduler": {
                "iterations_total": self.iterations_total,
                "mean_batch_size": sum(sizes) / len(sizes) if sizes else 0.0,
                "max_batch_size": max(sizes, default=0),
            },
        }
