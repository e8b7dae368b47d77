"""GPU: the engine's step function against the plain implementation, in float32
and in bfloat16, for every way of cutting and batching the same requests."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen2
import replay_util
from conftest import ROOT, random_tokens

pytestmark = pytest.mark.gpu

# float32: sums of a few hundred float32 products in another order than torch's.
F32_TOL = dict(rtol=1e-4, atol=2e-5)
# bfloat16: activations are rounded to 8 mantissa bits between kernels while the
# plain implementation keeps float32; the reference allows rtol=atol=2e-2 for its
# 16-bit path (tests/remote_gpu_tests.py:117).
BF16_TOL = dict(rtol=2e-2, atol=2e-2)
TOL = {"float32": F32_TOL, "bfloat16": BF16_TOL}

LENGTHS = {"A": [5, 17, 33, 70, 100], "B": [1, 9, 40, 64, 100, 131], "C": [3, 30, 77, 48]}


def make_requests(name: str, raw: dict) -> dict[str, list[int]]:
    return {f"{name}{i}": random_tokens(n, raw["vocab_size"], seed=100 + i) for i, n in enumerate(LENGTHS[name])}


def plain_all(raw, tensors, requests):
    weights = {k: v.float() for k, v in tensors.items()}
    return {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}


def make_runner(folder, dtype, kv_tokens, page_size, max_running=8, graph_decode=False):
    from cie_amd.config import build_engine_config
    from cie_amd.engine import Runner, load_model

    model, config = load_model(folder, dtype, "cuda:0")
    engine_config = build_engine_config(
        dtype=dtype, page_size=page_size, kv_tokens=kv_tokens, max_running=max_running,
        max_model_len=min(config.max_position_embeddings, kv_tokens), prefix_cache_pages=0, graph_decode=graph_decode)
    return Runner(model, engine_config, "cuda:0")


_ROUGH: dict = {}


def rough_all(name, tiny_folders, requests):
    """The plain implementation in bfloat16 throughout, once per configuration."""
    if name not in _ROUGH:
        _, raw, tensors = tiny_folders[name]
        weights = {k: v.float() for k, v in tensors.items()}
        _ROUGH[name] = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16)
                        for rid, tokens in requests.items()}
    return _ROUGH[name]


@pytest.fixture(scope="module")
def plain(tiny_folders):
    out = {}
    for name, (folder, raw, tensors) in tiny_folders.items():
        requests = make_requests(name, raw)
        out[name] = (requests, plain_all(raw, tensors, requests))
    return out


SCHEDULES = {
    "whole": replay_util.whole,
    "tail": replay_util.tail_one_by_one,
    "portions": replay_util.portions,
    "mixed": lambda requests: replay_util.mixed(requests, live=4),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_replay_matches_plain(tiny_folders, plain, name, schedule, dtype):
    folder, raw, _ = tiny_folders[name]
    requests, expected = plain[name]
    steps = SCHEDULES[schedule](requests)
    page = 16 if name == "A" else 8
    # exactly as many pages as the live requests need: finished requests' pages are used again
    pool = replay_util.max_live_tokens(steps, page=page)
    print(f"case {name} {schedule} {dtype}: {len(steps)} steps, pool {pool} tokens", flush=True)
    runner = make_runner(folder, dtype, pool, page)
    outputs = replay_util.drive_runner(runner, steps)
    rows = replay_util.by_position(steps, outputs)
    worst = replay_util.compare(rows, expected, **TOL[dtype])
    print(f"worst |diff| {worst:.3e}", flush=True)
    if dtype == "bfloat16":
        # the stricter yardstick: closer to the float32 logits than the plain model run in bfloat16 is
        print("rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
              % replay_util.closer_than_plain_bfloat16(rows, expected, rough_all(name, tiny_folders, requests)), flush=True)
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("page", [16, 64])
def test_replay_with_the_four_wave_prompt_attention(tiny_folders, plain, monkeypatch, schedule, page):
    """Pages of 16 keys and more send prompt portions to the attention form in which
    four waves share a tile's keys (Tiny-B: head size 32, three heads per group)."""
    from cie_amd.kernels import ops

    seen = []
    real = ops.paged_attention_mfma

    def spy(*args, **kwargs):
        seen.append(kwargs.get("tile_waves", 1))
        return real(*args, **kwargs)

    monkeypatch.setattr(ops, "paged_attention_mfma", spy)
    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    steps = SCHEDULES[schedule](requests)
    pool = replay_util.max_live_tokens(steps, page=page)
    runner = make_runner(folder, "bfloat16", pool, page)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL["bfloat16"])
    assert ops.TILE_WAVES in seen
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("heads", [(16, 2), (28, 4), (10, 2)])
@pytest.mark.parametrize("rows", [128, 64])
def test_replay_with_the_prompt_attention_that_shares_keys_through_lds(tmp_path, monkeypatch, schedule, heads, rows):
    """Prompt portions of many rows go to tiles of 128 rows and eight waves, or of 64 rows and four, whose keys
    and values pass through LDS (heads of 128 dimensions).  The tiny requests here never have that many rows:
    the thresholds are set so that every portion takes that form in the one size or the other, with groups of
    8, 7 and 5 heads (tiles of 16, 18 and 25 tokens, or 8, 9 and 12)."""
    from conftest import TINY_C, make_folder
    from cie_amd.kernels import ops
    from cie_amd.parts import attention

    monkeypatch.setattr(attention, "EIGHT_WAVE_TILES", 0)  # (a share of the compute units: any tile at all)
    monkeypatch.setattr(attention, "LARGE_TILES_ABOVE", -1 if rows == 128 else 1e9)
    seen = []
    real = ops.paged_attention_mfma

    def spy(*args, **kwargs):
        seen.append(kwargs.get("tile_waves", 1))
        if kwargs.get("tile_waves", 1) == ops.PROMPT_WAVES:
            assert 16 * kwargs["row_tiles"] == rows
        return real(*args, **kwargs)

    monkeypatch.setattr(ops, "paged_attention_mfma", spy)
    q_heads, kv_heads = heads
    raw = dict(TINY_C, hidden_size=128, num_attention_heads=q_heads, num_key_value_heads=kv_heads, head_dim=128,
               intermediate_size=96, vocab_size=211, eos_token_id=1, attention_bias=True)
    folder, tensors = make_folder(tmp_path, raw, seed=5)
    requests = {f"r{i}": random_tokens(n, 211, seed=80 + i) for i, n in enumerate((9, 47, 130, 200))}
    expected = plain_all(raw, tensors, requests)
    steps = SCHEDULES[schedule](requests)
    runner = make_runner(folder, "bfloat16", replay_util.max_live_tokens(steps, page=16), 16, max_running=4)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    weights = {k: v.float() for k, v in tensors.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    print(heads, schedule, "rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
          % replay_util.closer_than_plain_bfloat16(rows, expected, rough), flush=True)
    assert ops.PROMPT_WAVES in seen
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("graph", [False, True])
def test_replay_with_the_four_wave_decode_attention(tiny_folders, plain, monkeypatch, graph):
    """Decode rows go to the four-wave attention form only for long contexts and not for
    a few sequences; make every context long enough and every batch large enough, eagerly
    and in captured steps."""
    from cie_amd.kernels import ops
    from cie_amd.parts import attention

    monkeypatch.setattr(attention, "WIDE_DECODE_KEYS", 0)
    monkeypatch.setattr(attention, "FEW_DECODE_UNITS", 0)
    seen = []
    real = ops.paged_attention_mfma

    def spy(*args, **kwargs):
        seen.append((kwargs["tokens_per_tile"], kwargs.get("tile_waves", 1), kwargs.get("n_splits", 1)))
        return real(*args, **kwargs)

    monkeypatch.setattr(ops, "paged_attention_mfma", spy)
    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    steps = replay_util.mixed(requests, live=4, decode_tail=30, seed=8)
    runner = make_runner(folder, "bfloat16", replay_util.max_live_tokens(steps, page=16), 16, graph_decode=graph)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL["bfloat16"])
    assert any(per_tile == 1 and waves == ops.TILE_WAVES for per_tile, waves, _ in seen), seen[:8]
    if graph:  # captured steps size their parts for the longest request the engine takes: more than one part
        assert any(per_tile == 1 and waves == ops.TILE_WAVES and splits > 1 for per_tile, waves, splits in seen), seen[:8]
        assert runner.graph_replays >= 20


def test_logits_of_a_captured_step_are_the_callers_to_keep(tiny_folders):
    """A captured decode step writes into a buffer of its graph's; what ``run`` returns must not change
    when the same graph is replayed for the next step."""
    folder, raw, _ = tiny_folders["A"]
    tokens = random_tokens(20, raw["vocab_size"], seed=77)
    from cie_amd.engine.runner import StepEntry

    runner = make_runner(folder, "bfloat16", 64, 16, graph_decode=True)
    runner.cache.admit("k")
    runner.run([StepEntry("k", tokens[:18], 0, ())])
    first = runner.run([StepEntry("k", tokens[18:19], 18, (0,))])
    kept = first.cpu().clone()
    second = runner.run([StepEntry("k", tokens[19:20], 19, (0,))])
    assert runner.graph_replays == 2
    assert torch.equal(first.cpu(), kept) and not torch.equal(second.cpu(), kept)
    runner.cache.release("k")


ODD_SIZES = [  # hidden, heads, kv heads, head_dim, intermediate, vocabulary
    (75, 3, 1, 16, 77, 97),      # an odd width: no 16-byte rows anywhere
    (90, 6, 2, 48, 50, 1001),
    (34, 2, 2, 80, 33, 130),     # heads wider than the model
    (200, 24, 8, 16, 12, 50),    # many small heads, a feed-forward narrower than a tile
    (30, 3, 1, 8, 50, 101),      # the smallest head the kernels take
    (64, 2, 1, 136, 12, 50),     # a head size in steps of 8 that the matrix-core attention does not take
    (128, 2, 1, 256, 64, 300),   # the widest head
]


HEAD_SIZES = [  # head sizes and group sizes the matrix-core attention takes (pages of 16 tokens: its four-wave forms)
    (64, 2, 1, 32, 40, 97),      # two heads on one key head
    (192, 3, 3, 64, 100, 300),   # no grouping
    (96, 7, 1, 96, 64, 211),     # seven heads on one key head: rows of a tile that are no power of two
    (256, 16, 2, 128, 300, 515),
    (128, 10, 2, 64, 72, 130),   # groups of five
    (512, 16, 1, 32, 64, 97),    # sixteen heads on one key head: a tile's rows are one token
    (160, 40, 8, 128, 96, 130),  # forty heads on eight key heads (groups of five at the widest common head size)
]


@pytest.mark.parametrize("schedule", ["portions", "mixed"])
@pytest.mark.parametrize("sizes", HEAD_SIZES, ids=lambda s: "x".join(map(str, s)))
def test_replay_at_the_head_sizes_of_the_matrix_core_attention(tmp_path, sizes, schedule):
    """bfloat16 with pages of 16 tokens, where prompt portions and decode rows take the tiled attention
    forms (and, side by side, one launch for both): portions of changing size and a mixed schedule with
    reused pages at several head and group sizes, to the plain model's logits."""
    from conftest import TINY_C, make_folder

    hidden, heads, kv_heads, head_dim, intermediate, vocab = sizes
    raw = dict(TINY_C, hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
               intermediate_size=intermediate, vocab_size=vocab, eos_token_id=1, attention_bias=True)
    folder, tensors = make_folder(tmp_path, raw, seed=4)
    requests = {f"r{i}": random_tokens(n, vocab, seed=60 + i) for i, n in enumerate((9, 47, 130, 200))}
    expected = plain_all(raw, tensors, requests)
    steps = SCHEDULES[schedule](requests)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = make_runner(folder, "bfloat16", pool, 16, max_running=4)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    # (peaked softmaxes at widths of hundreds: the yardstick is the plain implementation run in bfloat16)
    weights = {k: v.float() for k, v in tensors.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    print(sizes, schedule, "rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
          % replay_util.closer_than_plain_bfloat16(rows, expected, rough), flush=True)
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", ODD_SIZES, ids=lambda s: "x".join(map(str, s)))
def test_replay_at_odd_sizes(tmp_path, sizes, dtype):
    """Widths, head sizes and vocabularies that no fast path was written for run through the kernels
    that take every size, in a mixed schedule with reused pages, to the plain model's logits."""
    from conftest import TINY_C, make_folder

    hidden, heads, kv_heads, head_dim, intermediate, vocab = sizes
    raw = dict(TINY_C, hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
               intermediate_size=intermediate, vocab_size=vocab, eos_token_id=1)
    folder, tensors = make_folder(tmp_path, raw, seed=3)
    requests = {f"r{i}": random_tokens(n, vocab, seed=50 + i) for i, n in enumerate((5, 33, 70))}
    expected = plain_all(raw, tensors, requests)
    steps = replay_util.mixed(requests, live=3)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = make_runner(folder, dtype, pool, 16, max_running=4)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL[dtype])
    assert runner.cache.stats().pages_used == 0


def test_a_head_size_the_kernels_do_not_take_is_refused_when_the_model_is_built(tmp_path):
    from conftest import TINY_C
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors

    for head_dim in (20, 264):
        config = config_from_dict(dict(TINY_C, head_dim=head_dim))
        with pytest.raises(ValueError, match="head_dim must be a multiple of 8 up to 256"):
            expected_tensors(config.model_spec())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_captured_steps_with_prompt_portions_match_plain(tiny_folders, plain, name, dtype):
    """Steps that bring prompt portions beside decode tokens are captured when their shape comes a second
    time and replayed from then on, with other tokens, slots, pages and lengths at every replay (pages of
    finished requests are used again): every wanted row against the plain model, and against the same
    schedule run launch by launch."""
    folder, raw, _ = tiny_folders[name]
    requests, expected = plain[name]
    page = 16 if name == "A" else 8
    steps = replay_util.fixed_portions(requests, portion=8 if name == "B" else 5)
    pool = replay_util.max_live_tokens(steps, page=page)
    runner = make_runner(folder, dtype, pool, page, graph_decode=True)
    assert runner.mixed_graphs is not None
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, every_position=False, **TOL[dtype])
    assert runner.mixed_graph_captures >= 2 and runner.mixed_graph_replays >= 8, (
        runner.mixed_graph_captures, runner.mixed_graph_replays)
    assert runner.cache.stats().pages_used == 0
    eager = make_runner(folder, dtype, pool, page, graph_decode=False)
    assert eager.mixed_graphs is None
    eager_rows = replay_util.by_position(steps, replay_util.drive_runner(eager, steps))
    for rid, positions in rows.items():
        for position, row in positions.items():
            if dtype == "float32":  # the same kernels on the same rows: the same bits
                assert np.array_equal(row, eager_rows[rid][position]), (rid, position)
            else:  # (the parts of a portion's keys may be cut elsewhere)
                np.testing.assert_allclose(row, eager_rows[rid][position], **TOL[dtype])


def test_shapes_beyond_the_limit_drop_the_least_recently_used(tiny_folders, plain):
    from cie_amd.config import build_engine_config
    from cie_amd.engine import Runner, load_model

    folder, raw, _ = tiny_folders["A"]
    requests, expected = plain["A"]
    model, config = load_model(folder, "float32", "cuda:0")
    steps = replay_util.fixed_portions(requests, portion=5)
    pool = replay_util.max_live_tokens(steps, page=16)
    runner = Runner(model, build_engine_config(dtype="float32", page_size=16, kv_tokens=pool, max_running=8,
                                               max_model_len=min(config.max_position_embeddings, pool), prefix_cache_pages=0,
                                               graph_mixed_steps=1), "cuda:0")
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, every_position=False, **TOL["float32"])
    assert len(runner.mixed_graphs.steps) == 1 and runner.mixed_graph_captures >= 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_captured_decode_steps_match_plain(tiny_folders, plain, name, dtype):
    """Decode steps replayed from captured graphs (buckets 1, 2 and 4, padded
    rows on the pad slot), between eager prompt portions, every replay checked:
    the tail schedule decodes one request at a time, the mixed one several."""
    folder, raw, _ = tiny_folders[name]
    requests, expected = plain[name]
    page = 16 if name == "A" else 8
    schedules = {"tail": replay_util.tail_one_by_one,
                 "mixed": lambda r: replay_util.mixed(r, live=4, decode_tail=30, seed=5)}
    for schedule, build in schedules.items():
        steps = build(requests)
        pool = replay_util.max_live_tokens(steps, page=page)
        runner = make_runner(folder, dtype, pool, page, graph_decode=True)
        assert runner.graphs is not None
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        replay_util.compare(rows, expected, **TOL[dtype])
        assert runner.graph_replays >= 20 and runner.graph_captures >= (1 if schedule == "tail" else 2)
        print(f"{name} {schedule} {dtype}: {runner.graph_captures} captures, {runner.graph_replays} replays", flush=True)


@pytest.mark.parametrize("graph", [False, True])
def test_many_decoding_requests_run_the_library_products(tiny_folders, plain, graph):
    """More than 16 rows in a step send the products to the vendor library (and, with
    17 to 64 rows, the down product to the split-K kernel for 32 and 64 rows); with
    graphs on, the library calls are inside the captured steps and every replay is
    checked.  24 requests live at once, decoded side by side for 30 steps."""
    folder, raw, tensors = tiny_folders["B"]
    lengths = [40 + (7 * i) % 23 for i in range(24)]
    requests = {f"m{i}": random_tokens(n, raw["vocab_size"], seed=300 + i) for i, n in enumerate(lengths)}
    expected = plain_all(raw, tensors, requests)
    steps = replay_util.mixed(requests, live=24, chunk_sizes=(9, 4, 13), decode_tail=30, seed=9)
    assert max(len(step["entries"]) for step in steps) > 16
    pool = replay_util.max_live_tokens(steps, page=8)
    runner = make_runner(folder, "bfloat16", pool, 8, max_running=24, graph_decode=graph)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL["bfloat16"])
    if graph:
        assert runner.graph_replays >= 10 and max(runner.graphs.buckets) == 32


@pytest.mark.parametrize("graph", [False, True])
def test_products_cut_along_k_match_plain(tiny_folders, plain, monkeypatch, graph):
    """The decode products that cut a long K into parts (summed by the next norm
    kernel) only engage at sizes the tiny models do not have; force them."""
    from cie_amd.parts import linear

    monkeypatch.setattr(linear, "PART_K", 128)  # Tiny-B's down product has K = 328: three parts
    monkeypatch.setattr(linear, "PART_MIN_K", 256)
    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    steps = replay_util.mixed(requests, live=4, decode_tail=30, seed=6)
    runner = make_runner(folder, "bfloat16", replay_util.max_live_tokens(steps, page=8), 8, graph_decode=graph)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL["bfloat16"])


@pytest.mark.parametrize("graph", [False, True])
def test_steps_queued_behind_a_busy_gpu_keep_their_own_metadata(tiny_folders, plain, graph):
    """The host may run many steps ahead of the GPU (prompt portions of a large model want no logits,
    so nothing makes the host wait).  Each step's token ids, positions and table rows must then still be
    the step's own when its copy finally runs: here the GPU is kept busy while portions of different
    sizes, decode steps and a slot that changes hands are queued, and only the end is checked."""
    from cie_amd.engine.runner import StepEntry

    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    runner = make_runner(folder, "float32", 512, 8, graph_decode=graph)
    if graph:
        runner.warm_up()
    long_one, short_one, other = requests["B5"], requests["B2"], requests["B3"]  # 131, 40 and 64 tokens
    runner.cache.admit("x"), runner.cache.admit("y")
    torch.cuda.synchronize()
    torch.cuda._sleep(int(1.5e9))  # the GPU spins for most of a second: everything below queues up behind it
    fed = {"x": 0, "y": 0}

    def step(*portions):
        entries = []
        for rid, tokens, count in portions:
            entries.append(StepEntry(rid, tokens[fed[rid]: fed[rid] + count], fed[rid], []))
            fed[rid] += count
        runner.run(entries)

    step(("x", long_one, 7))
    step(("x", long_one, 33), ("y", short_one, 20))
    step(("x", long_one, 2))
    step(("y", short_one, 19), ("x", long_one, 16))
    for _ in range(6):  # single tokens: captured steps when graphs are on
        step(("x", long_one, 1))
    runner.cache.release("y")  # its slot goes to another request while the copies above are still queued
    runner.cache.admit("z")
    fed["z"] = 0
    step(("z", other, 50), ("x", long_one, 40))
    step(("x", long_one, 2))
    last_x = runner.run([StepEntry("x", long_one[fed["x"]:], fed["x"], [len(long_one) - fed["x"] - 1])])
    last_z = runner.run([StepEntry("z", other[50:], 50, [len(other) - 51])])
    torch.testing.assert_close(last_x[0].cpu(), expected["B5"][-1], **F32_TOL)
    torch.testing.assert_close(last_z[0].cpu(), expected["B3"][-1], **F32_TOL)


def test_mixed_reuses_pages(tiny_folders, plain):
    """The mixed schedule as the replays run it (four live requests, a pool of exactly the peak): the
    engine's allocator hands pages that one request gave back to a later one, while other requests are
    in the middle of their sequences, and the logits written through those pages are the plain model's."""
    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    steps = replay_util.mixed(requests, live=4)
    pool = replay_util.max_live_tokens(steps, page=8)
    assert pool < sum(-(-len(t) // 8) * 8 for t in requests.values())
    runner = make_runner(folder, "float32", pool, 8)
    allocator = runner.cache.groups[0].allocator
    owners: dict[int, list[str]] = {}
    real = allocator.allocate

    def spy(holder, n_pages):
        pages = real(holder, n_pages)
        for page in pages:
            owners.setdefault(page, []).append(holder)
        return pages

    allocator.allocate = spy
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **F32_TOL)
    reused = {page: who for page, who in owners.items() if len(set(who)) > 1}
    assert len(reused) >= 4, f"pages handed to a second request: {reused}"
    assert sum(len(who) for who in owners.values()) > allocator.total_pages, "more pages handed out than the pool has"
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tiny_folders, plain, tmp_path, dtype):
    """bin/trace_run end to end: JSON lines in, <step>.f32 files and 'done' lines out."""
    folder, raw, _ = tiny_folders["B"]
    requests, expected = plain["B"]
    steps = replay_util.mixed(requests, live=4, seed=3)
    pool = replay_util.max_live_tokens(steps, page=64)
    out_dir = tmp_path / "out"
    # (first a step whose only request brings nothing and ends: it is answered and leaves no file)
    idle = {"step": 999, "entries": [{"id": "ghost", "tokens": [], "want": []}], "end": ["ghost"]}
    text = "\n".join(json.dumps(step) for step in [idle] + steps) + "\n"
    done = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
         "--out", str(out_dir), "--max-tokens", str(pool)],
        input=text, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    lines = [line for line in done.stdout.splitlines() if line.startswith("done ")]
    assert lines == ["done 999"] + [f"done {step['step']}" for step in steps]
    assert not (out_dir / "999.f32").exists()
    vocab = raw["vocab_size"]
    outputs = {}
    for step in steps:
        path = out_dir / f"{step['step']}.f32"
        wanted = sum(len(e["want"]) for e in step["entries"])
        if wanted:
            data = np.fromfile(path, dtype="<f4")
            assert data.size == wanted * vocab
            outputs[step["step"]] = data.reshape(wanted, vocab)
        else:
            assert not path.exists()
    rows = replay_util.by_position(steps, outputs)
    replay_util.compare(rows, expected, **TOL[dtype])


def test_trace_run_takes_many_short_requests_and_names_a_step_that_does_not_fit(tiny_folders, plain, tmp_path):
    """Fourteen requests live at once, each well inside the token bound: the program has a slot for every
    page of its pool.  A step that the pool cannot hold ends the run with a message that names the step."""
    folder, raw, tensors = tiny_folders["A"]
    weights = {k: v.float() for k, v in tensors.items()}
    requests = {f"s{i}": random_tokens(3 + i % 4, raw["vocab_size"], seed=900 + i) for i in range(14)}
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": tokens[:2], "want": [1]} for rid, tokens in requests.items()],
              "end": []},
             {"step": 1, "entries": [{"id": rid, "tokens": tokens[2:], "want": list(range(len(tokens) - 2))}
                                     for rid, tokens in requests.items()], "end": list(requests)}]
    pool = replay_util.max_live_tokens(steps, page=64)
    out_dir = tmp_path / "out"
    text = "\n".join(json.dumps(step) for step in steps) + "\n"
    command = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
               "--out", str(out_dir)]
    done = subprocess.run(command + ["--max-tokens", str(pool)], input=text, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done ")] == ["done 0", "done 1"]
    vocab = raw["vocab_size"]
    outputs = {n: np.fromfile(out_dir / f"{n}.f32", dtype="<f4").reshape(-1, vocab) for n in (0, 1)}
    rows = replay_util.by_position(steps, outputs)
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    replay_util.compare(rows, expected, every_position=False, **F32_TOL)
    # too small a pool (pages of 8: two pages hold two requests) and too few slots: a message, not a traceback
    for extra in (["--max-tokens", "16", "--page-size", "8"], ["--max-tokens", str(pool), "--max-requests", "5"]):
        short = subprocess.run(command + extra, input=text, capture_output=True, text=True, timeout=600)
        assert short.returncode == 1 and "step 0 does not fit" in short.stderr and "Traceback" not in short.stderr, \
            short.stderr[-2000:]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,layers,vocab", [("0.5b", 2, None), ("3b", 1, None), ("7b", 1, 20011), ("14b", 1, 20011), ("72b", 1, 8209)])
def test_replay_at_the_sizes_of_real_models(tmp_path_factory, shape, layers, vocab, dtype):
    """The widths, head counts and vocabulary of models of the family (few layers,
    random weights; the largest with a short vocabulary, to keep its files small): the
    kernels meet the shapes that serving meets, not only the tiny ones.  One request most of it at once and its tail token by token, another
    in portions beside it; logits at the end of every step against the plain
    implementation."""
    from conftest import make_folder
    from cie_amd.workloads import SHAPES

    raw = dict(SHAPES[shape], architectures=["Qwen2ForCausalLM"], num_hidden_layers=layers)
    if vocab is not None:
        raw.update(vocab_size=vocab, eos_token_id=vocab - 1)
    # (at these widths the tiny models' factor of 8 on the query and key weights would make every softmax
    # one-hot, and a bfloat16 rounding of a score could then swap the key it picks)
    folder, tensors = make_folder(tmp_path_factory.mktemp(f"real_{shape}"), raw, seed=31, factor=1.5)
    requests = {"long": random_tokens(190, raw["vocab_size"], seed=7), "cut": random_tokens(121, raw["vocab_size"], seed=8)}
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    # what float32 itself costs at these widths: the plain implementation with float64 layers
    exact = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.float64) for rid, tokens in requests.items()}
    del weights
    steps = []

    def step(entries, end=()):
        steps.append({"step": len(steps), "end": list(end),
                      "entries": [{"id": rid, "tokens": tokens, "want": [len(tokens) - 1]} for rid, tokens in entries]})

    long, cut = requests["long"], requests["cut"]
    step([("long", long[:149])])
    step([("long", [long[149]]), ("cut", cut[:64])])  # 65 rows: a second row block for the products of few rows
    fed = 64
    for i, size in enumerate((33, 2, 17, 5)):  # the other request's portions beside single tokens of the first
        step([("long", [long[150 + i]]), ("cut", cut[fed:fed + size])], end=["cut"] if fed + size == len(cut) else [])
        fed += size
    assert fed == len(cut)
    for i in range(154, len(long)):
        step([("long", [long[i]])], end=["long"] if i == len(long) - 1 else [])
    runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=16), 16)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    if dtype == "float32":
        # sums of thousands of float32 products: the engine may be as far from the exact logits as a few times
        # what the plain float32 implementation is (its sums run in another order)
        plain_error = max(float((expected[rid] - exact[rid]).abs().max()) for rid in requests)
        print(f"plain float32 against float64 layers: {plain_error:.3e}", flush=True)
        worst = replay_util.compare(rows, exact, every_position=False, rtol=0.0, atol=4 * plain_error + 1e-6)
        print(f"{shape} x {layers} layers float32: worst |diff| to exact {worst:.3e}, plain float32 {plain_error:.3e}", flush=True)
    else:
        # bfloat16 keeps 8 bits, and at these widths a logit sums 896 to 2,048 rounded values: what that costs is
        # measured, not assumed: the plain implementation run in bfloat16 throughout is the yardstick, and the
        # engine (float32 residual stream, softmax and sums) has to be closer to the float32 logits than it is
        weights = {k: v.float() for k, v in tensors.items()}
        rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
        del weights
        rms, worst, plain_rms, plain_worst = replay_util.closer_than_plain_bfloat16(rows, expected, rough)
        print(f"{shape} x {layers} layers bfloat16: root mean square {rms:.3e} (plain in bfloat16 {plain_rms:.3e}), "
              f"worst {worst:.3e} ({plain_worst:.3e})", flush=True)
    assert runner.cache.stats().pages_used == 0


def test_replay_with_the_keys_of_prompt_portions_cut(tiny_folders, monkeypatch):
    """A short portion behind a long context has few tiles and many keys: its keys are cut
    into parts that a second kernel joins (Tiny-B, the limit lowered so that 300 positions reach it)."""
    from cie_amd.kernels import ops
    from cie_amd.parts import attention

    monkeypatch.setattr(attention, "PROMPT_SPLIT_KEYS", 64)
    seen = []
    real = ops.paged_attention_mfma

    def spy(*args, **kwargs):
        seen.append((kwargs.get("tokens_per_tile", 1), kwargs.get("n_splits", 1)))
        return real(*args, **kwargs)

    monkeypatch.setattr(ops, "paged_attention_mfma", spy)
    folder, raw, tensors = tiny_folders["B"]
    requests = {"r": random_tokens(300, raw["vocab_size"], seed=77), "s": random_tokens(150, raw["vocab_size"], seed=78)}
    expected = plain_all(raw, tensors, requests)
    steps, fed = [], {"r": 0, "s": 0}

    def step(parts, end=()):
        entries = []
        for rid, size in parts:
            tokens = requests[rid][fed[rid]: fed[rid] + size]
            fed[rid] += size
            entries.append({"id": rid, "tokens": tokens, "want": list(range(len(tokens)))})
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    step([("r", 200)])
    step([("r", 60), ("s", 120)])     # portions of two requests with different contexts in one step
    step([("r", 38), ("s", 1)])       # beside a single token
    step([("r", 2), ("s", 29)], end=["r", "s"])
    runner = make_runner(folder, "bfloat16", replay_util.max_live_tokens(steps, page=16), 16)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, expected, **TOL["bfloat16"])
    assert any(per_tile > 1 and splits > 1 for per_tile, splits in seen), seen
    assert runner.cache.stats().pages_used == 0


@pytest.fixture(scope="module")
def long_context_case(tmp_path_factory):
    """(folder, raw, requests, plain float32 logits, plain bfloat16 logits) of the 6,040-token case, made once."""
    from conftest import make_folder

    raw = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=256, num_hidden_layers=2,
               num_attention_heads=4, num_key_value_heads=1, head_dim=128, intermediate_size=520, vocab_size=1003,
               rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=8192, tie_word_embeddings=True,
               attention_bias=True, use_sliding_window=False, eos_token_id=1002)
    folder, tensors = make_folder(tmp_path_factory.mktemp("long_context"), raw, seed=41, factor=6.0)
    requests = {"long": random_tokens(6040, raw["vocab_size"], seed=17), "short": random_tokens(90, raw["vocab_size"], seed=18)}
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    return folder, raw, requests, expected, rough


@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_replay_of_a_context_of_six_thousand_tokens(long_context_case, dtype, graphs):
    """Thousands of keys behind a token, through the engine and not only through the attention kernel: a prompt of
    6,000 tokens in portions of up to 2,048 (the later ones behind thousands of keys, their keys cut into parts), its
    last tokens one by one beside another request's portion and single tokens (keys of a single token cut into
    parts by the longest context of the step).  Heads of 128 as in the family's models, queries and keys scaled so
    that a token attends to a few keys anywhere in its context: a lost or misplaced block of far keys moves the logits.
    Once more with the steps of single tokens replayed from a captured graph."""
    folder, raw, requests, expected, rough = long_context_case
    long, short = requests["long"], requests["short"]
    steps = []

    def step(entries, end=()):
        steps.append({"step": len(steps), "end": list(end),
                      "entries": [{"id": rid, "tokens": tokens, "want": want} for rid, tokens, want in entries]})

    step([("long", long[:2048], [0, 1000, 2047])])
    step([("long", long[2048:4096], [0, 2047])])
    step([("long", long[4096:5990], [3, 1893])])
    step([("long", long[5990:6000], list(range(10))), ("short", short[:50], [49])])  # a short portion behind 5,990 keys
    for i in range(40):
        step([("long", [long[6000 + i]], [0]), ("short", [short[50 + i]], [0])], end=["long", "short"] if i == 39 else [])
    runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=16), 16, graph_decode=graphs)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    assert len(rows["long"]) == 3 + 2 + 2 + 10 + 40 and len(rows["short"]) == 41
    if graphs:
        assert runner.graph_captures == 1 and runner.graph_replays >= 39, (runner.graph_captures, runner.graph_replays)
    if dtype == "float32":
        worst = replay_util.compare(rows, expected, every_position=False, **F32_TOL)
        print(f"6,040 tokens float32: worst |diff| {worst:.3e}", flush=True)
    else:
        print("6,040 tokens bfloat16: rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
              % replay_util.closer_than_plain_bfloat16(rows, expected, rough), flush=True)
    assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("seed", range(12))
def test_random_traces_match_plain(tiny_folders, seed):
    """Requests of random lengths fed in random cuts (single tokens, pairs, up to a page's edge, one past it,
    anything), up to four live, some left out of a step, logits wanted at random places, in a pool of exactly the
    live requests' pages, eager or from captured graphs: float32 within the tolerance of the fixed schedules;
    bfloat16, row by row, no further from the float32 logits than 1.5 times what the plain implementation run in
    bfloat16 is at that row (or the fixed tolerance, where that is larger)."""
    import random

    rng = random.Random(1000 + seed)
    name = "ABC"[seed % 3]
    folder, raw, tensors = tiny_folders[name]
    page = rng.choice([16, 64]) if name == "A" else rng.choice([8, 16, 64])
    lengths = [rng.randint(1, raw["max_position_embeddings"]) for _ in range(rng.randint(2, 7))]
    requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"], page)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    for dtype in ("float32", "bfloat16"):
        graphs = rng.random() < 0.5
        print(f"case {name} page {page} {dtype} graphs {graphs}: lengths {lengths}, {len(steps)} steps", flush=True)
        runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=page), page, graph_decode=graphs)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        if dtype == "float32":
            replay_util.compare(rows, {rid: expected[rid] for rid in rows}, every_position=False, **F32_TOL)
        else:
            for rid, by_position in rows.items():
                for position, row in by_position.items():
                    off = float((torch.from_numpy(row) - expected[rid][position]).abs().max())
                    plain_off = float((rough[rid][position].float() - expected[rid][position]).abs().max())
                    assert off <= max(BF16_TOL["atol"], 1.5 * plain_off), (rid, position, off, plain_off)
        assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("shape,seed", [("0.5b", 49), ("3b", 54), ("7b", 48), ("14b", 50)])
def test_random_traces_at_the_sizes_of_real_models(tmp_path_factory, shape, seed):
    """Random cuts at the widths and heads that serving meets (one layer, a short vocabulary): steps of one row to
    several hundred meet the hand-written products of few rows, those whose waves share the rows, the library's,
    and both attention forms.  Float32 against float64 layers within four times the plain float32 implementation's
    own distance; bfloat16 closer to the float32 logits than the plain implementation run in bfloat16."""
    import random

    from conftest import make_folder
    from cie_amd.workloads import SHAPES

    raw = dict(SHAPES[shape], architectures=["Qwen2ForCausalLM"], num_hidden_layers=2 if shape == "0.5b" else 1,
               vocab_size=4099, eos_token_id=4098)
    folder, tensors = make_folder(tmp_path_factory.mktemp(f"random_{shape}"), raw, seed=31, factor=1.5)
    rng = random.Random(seed)
    page = rng.choice([16, 64])
    lengths = [rng.choice([rng.randint(1, 40), rng.randint(1, 200), rng.randint(100, 700)]) for _ in range(rng.randint(3, 5))]
    requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"], page)
    print(f"{shape}: lengths {lengths}, {len(steps)} steps, most rows in a step "
          f"{max(sum(len(e['tokens']) for e in step['entries']) for step in steps)}", flush=True)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    exact = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.float64) for rid, tokens in requests.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    plain_error = max(float((expected[rid] - exact[rid]).abs().max()) for rid in requests)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=page), page, graph_decode=dtype == "bfloat16")
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        if dtype == "float32":
            replay_util.compare(rows, {rid: exact[rid] for rid in rows}, every_position=False, rtol=0.0, atol=4 * plain_error + 1e-6)
        else:
            replay_util.closer_than_plain_bfloat16(rows, expected, rough)
        assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("seed", [22, 32, 56, 94, 125, 142, 200, 201, 202, 203])
def test_random_configurations_and_traces(tmp_path_factory, seed):
    """A configuration drawn at random (head sizes from 16 to 256 in steps of 16, one to four key heads with one to
    eight query heads each, widths that are multiples of 2, 4 or 8 only, any vocabulary, one to three layers, bias
    or none, tied head or not, the norms' eps, the rotation's base) under a trace drawn at random: float32 against
    float64 layers within four times the plain float32 implementation's own distance, bfloat16 closer to the float32
    logits than the plain implementation run in bfloat16."""
    import random

    from conftest import make_folder

    rng = random.Random(seed)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 128, 160, 192, 256])
    kv_heads = rng.choice([1, 1, 2, 3, 4])
    q_heads = kv_heads * rng.choice([1, 2, 3, 4, 5, 7, 8])
    raw = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=rng.choice([2, 4, 8, 8]) * rng.randint(6, 60),
               num_hidden_layers=rng.randint(1, 3), num_attention_heads=q_heads, num_key_value_heads=kv_heads,
               head_dim=head_dim, intermediate_size=rng.choice([2, 8, 16]) * rng.randint(5, 60),
               vocab_size=rng.randint(40, 2500), rms_norm_eps=rng.choice([1e-6, 1e-5, 1e-3]),
               rope_theta=rng.choice([1e4, 1e6, 5e5]), max_position_embeddings=rng.randint(48, 400),
               tie_word_embeddings=rng.random() < 0.5, attention_bias=rng.random() < 0.7, use_sliding_window=False,
               eos_token_id=1)
    print({k: raw[k] for k in ("hidden_size", "num_attention_heads", "num_key_value_heads", "head_dim", "intermediate_size",
                               "vocab_size", "num_hidden_layers")}, flush=True)
    folder, tensors = make_folder(tmp_path_factory.mktemp(f"drawn_{seed}"), raw, seed=seed, factor=rng.choice([1.5, 4.0, 8.0]))
    page = rng.choice([4, 8, 16, 64])
    lengths = [rng.randint(1, raw["max_position_embeddings"]) for _ in range(rng.randint(2, 5))]
    requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"], page)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    exact = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.float64) for rid, tokens in requests.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    plain_error = max(float((expected[rid] - exact[rid]).abs().max()) for rid in requests)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=page), page, graph_decode=rng.random() < 0.5)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        if rows and dtype == "float32":
            replay_util.compare(rows, {rid: exact[rid] for rid in rows}, every_position=False, rtol=0.0, atol=4 * plain_error + 1e-6)
        elif rows:
            replay_util.closer_than_plain_bfloat16(rows, expected, rough)
        assert runner.cache.stats().pages_used == 0


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_traces_behind_thousands_of_keys(tmp_path_factory, seed):
    """One request of several thousand tokens (up to 14,000) and a few short ones under a trace drawn at random:
    portions of any length behind contexts of any length, single tokens whose keys are cut into parts, heads of 64
    and 128 with one to eight query heads a key head, queries and keys scaled so that far keys matter."""
    import random

    from conftest import make_folder

    rng = random.Random(seed)
    head_dim = rng.choice([64, 128, 128])
    kv_heads = rng.choice([1, 2])
    q_heads = kv_heads * rng.choice([1, 2, 4, 5, 8])
    longest = rng.choice([3000, 6000, 9000, 14000])
    raw = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=128, num_hidden_layers=rng.randint(1, 2),
               num_attention_heads=q_heads, num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=256,
               vocab_size=503, rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=longest + 64,
               tie_word_embeddings=True, attention_bias=True, use_sliding_window=False, eos_token_id=1)
    folder, tensors = make_folder(tmp_path_factory.mktemp(f"long_{seed}"), raw, seed=seed, factor=rng.choice([4.0, 6.0]))
    page = rng.choice([16, 16, 64])
    lengths = [rng.randint(longest // 2, longest)] + [rng.randint(1, 300) for _ in range(rng.randint(1, 3))]
    rng.shuffle(lengths)
    requests, steps = replay_util.random_trace(rng, lengths, raw["vocab_size"], page)
    print(f"heads {q_heads}/{kv_heads} x {head_dim}, lengths {lengths}, {len(steps)} steps", flush=True)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=page), page, graph_decode=rng.random() < 0.5)
        rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
        if dtype == "float32":
            replay_util.compare(rows, {rid: expected[rid] for rid in rows}, every_position=False, rtol=1e-4, atol=5e-5)
        else:
            replay_util.closer_than_plain_bfloat16(rows, expected, rough)
        assert runner.cache.stats().pages_used == 0
