"""The benchmark's contract with its driver: one GPU only, one JSON line with the agreed fields."""

from __future__ import annotations

import json
import subprocess
import sys

import pytest

from conftest import ROOT


def test_more_than_one_gpu_is_said_and_refused():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2", "--steps", "3", "--warmup", "1"],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    lines = done.stdout.strip().splitlines()
    assert len(lines) == 1 and "one GPU" in lines[0] and "--gpus 2" in lines[0]


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_fields():
    """A short run of one layer of the default shape: the line's fields, and that its figures follow from one another."""
    command = [sys.executable, str(ROOT / "bench.py"), "--gpus", "1", "--steps", "4", "--warmup", "1", "--layers", "1",
               "--context", "256", "--prefill-tokens", "64", "--mixed-portions", "6,20", "--long-contexts", ""]
    done = subprocess.run(command, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    lines = done.stdout.strip().splitlines()
    assert len(lines) == 1, lines
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert (line["n_gpus"], line["steps"], line["warmup"], line["dtype"]) == (1, 4, 1, "bf16")
    assert line["higher_is_better"] is True and line["unit"] == "tokens/s" and "synthetic" in line["data"]
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())  # flat
    assert (config["layers"], config["layers_full"], config["global_batch"], config["seq_len"]) == (1, 36, 8, 256)
    assert (config["hidden"], config["intermediate"], config["vocab"]) == (2048, 11008, 151936)
    # tokens a second of the median window = batch / its time per step
    assert line["value"] == pytest.approx(8 / (line["ms_per_step"] / 1e3), rel=0.02)
    roofline = line["roofline"]
    assert (roofline["bound"], roofline["peak"], roofline["unit"]) == ("hbm", 8000.0, "GB/s")
    assert roofline["frac"] == pytest.approx(roofline["achieved"] / roofline["peak"], abs=1e-3)
    prefill = line["prefill"]
    assert prefill["tokens"] == 64 and prefill["value"] == pytest.approx(64 / (prefill["ms"] / 1e3), rel=0.02)
    assert 0 < prefill["frac"] < 1 and 0 < roofline["frac"] < 1
    assert set(line["points"]) == {"decode_b1", "decode_b64"} and all(v > 0 for v in line["points"].values())
    # the steps that carry a prompt portion beside the decode tokens
    mixed = line["mixed"]
    assert (mixed["decoding"], mixed["context"]) == (8, 256)
    assert set(mixed["ms_per_step"]) == {"6", "20"} and all(v > 0 for v in mixed["ms_per_step"].values())
