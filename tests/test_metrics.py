"""The counters and latency windows (src/cloud_engine/metrics.py:19-31, 52-200 of the reference) and the
profiler ranges' switch (src/cloud_engine/profiling.py:10-26)."""

from __future__ import annotations

import random
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT
from cie_amd.metrics import Metrics, Window, quantile


def test_quantile_is_the_linear_interpolation_between_ranks():
    rng = random.Random(4)
    for count in (1, 2, 3, 10, 101):
        samples = [rng.uniform(-5, 50) for _ in range(count)]
        for fraction in (0.0, 0.25, 0.5, 0.95, 0.99, 1.0):
            assert quantile(samples, fraction) == pytest.approx(float(np.percentile(samples, 100 * fraction)), abs=1e-9)
    assert quantile([], 0.5) == 0.0
    assert quantile([3.0, 1.0, 2.0], 1.7) == 3.0 and quantile([3.0, 1.0, 2.0], -1) == 1.0  # fractions are clipped


def test_a_window_keeps_the_latest_samples():
    window = Window(4)
    for value in range(10):
        window.add(float(value))
    assert len(window) == 4
    summary = window.summary()
    assert summary["count"] == 4 and summary["p50"] == 7.5 and summary["p99"] == pytest.approx(8.97)


def test_snapshot_names_and_reset():
    metrics = Metrics(latency_samples=8, batch_samples=3)
    metrics.totals.completed += 2
    metrics.totals.output_tokens += 9
    metrics.first_token_ms.add(5.0)
    for requests, tokens in ((1, 10), (4, 4), (2, 7), (3, 3)):
        metrics.iteration(requests, tokens)
    snapshot = metrics.snapshot()
    assert snapshot["requests"] == {"completed_total": 2, "failed_total": 0, "cancelled_total": 0, "rejected_total": 0,
                                    "preempted_total": 0}
    assert snapshot["tokens"] == {"input_total": 24, "output_total": 9, "recomputed_total": 0}
    assert snapshot["scheduler"] == {"iterations_total": 4, "mean_batch_size": 3.0, "max_batch_size": 4}  # the latest three
    assert snapshot["latency_ms"]["ttft"] == {"count": 1, "p50": 5.0, "p95": 5.0, "p99": 5.0}
    metrics.reset()
    assert metrics.snapshot()["scheduler"]["iterations_total"] == 0 and len(metrics.first_token_ms) == 0


@pytest.mark.parametrize("switch", ["0", "1"])
def test_profiler_ranges_do_nothing_unless_switched_on(switch):
    """The switch is read once at import; off (or where torch cannot emit ranges, as without a GPU) every range is one
    shared object that does nothing; on, entering and leaving a range must still work."""
    code = ("import sys; sys.path.insert(0, %r); import cie_amd\n"
            "from cie_amd import profiling as p\n"
            "a, b = p.trace_range('x'), p.trace_range('y')\n"
            "with a:\n    with b:\n        pass\n"
            "print('shared' if a is b else 'marked')\n") % str(ROOT)
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                          env={**__import__("os").environ, "ENGINE_NVTX": switch})
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split()[-1] in (("shared",) if switch == "0" else ("shared", "marked"))
