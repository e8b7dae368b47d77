"""GPU: the engine against the plain implementation at the edges of what it says it runs: the longest
context a configuration allows (32,768 tokens), decode steps of 64 to 200 requests (the captured buckets of
64, 128 and 256 rows), and the smallest and largest pages."""

from __future__ import annotations

import random

import numpy as np
import pytest
import torch

import plain_qwen2
import replay_util
from conftest import make_folder, random_tokens, sharpen
from test_gpu_replay import BF16_TOL, F32_TOL, TOL, make_runner

pytestmark = pytest.mark.gpu


# ---------------------------------------------------------------------------------------------------------
# 32,768 tokens of context
# ---------------------------------------------------------------------------------------------------------

LONG = 32768
CHANNELS = 4
KEYS_PER_CHANNEL = 3
# where the planted keys lie: the first position, both sides of a page's and of a block's edge, both sides of the
# first portion's end, of a power of two in the middle, and the last position before the single tokens
KEY_POSITIONS = [0, 15, 16, 31, 32, 2048, 8191, 8192, 16401, 24575, 30001, LONG - 33]


def _planted_model(folder):
    """One layer, one key head of 128 dimensions under two query heads, width 128.  Beside random weights it
    has four *channels*: a token ``Y_c`` asks, through the slowest pair of rotated dimensions (which turns by
    0.04 rad over the whole context), for the keys of the tokens ``X_c,i`` and for little else: their scores
    stand some 8 above the largest of 32,000 random ones.  A key that a kernel loses (a block, a page, a
    part of the cut context) therefore moves the logits of the ``Y`` rows by a third of the attention's
    share, which also shows in bfloat16."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import RandomSource, write_tensors

    hidden, head_dim, vocab = 128, 128, 503
    raw = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=hidden, num_hidden_layers=1,
               num_attention_heads=2, num_key_value_heads=1, head_dim=head_dim, intermediate_size=256,
               vocab_size=vocab, rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=LONG,
               tie_word_embeddings=False, attention_bias=True, use_sliding_window=False, eos_token_id=1)
    expected = expected_tensors(config_from_dict(raw).model_spec())
    tensors = {k: v.float() for k, v in sharpen(RandomSource(77).load(expected, "float32", "cpu"), 5.0).items()}
    tensors["lm_head.weight"] *= 5.0  # logits of the order of one: the fixed tolerance of 16 bits then means something
    p = "model.layers.0.self_attn."
    key_tokens = [[vocab - 1 - (c * KEYS_PER_CHANNEL + i) for i in range(KEYS_PER_CHANNEL)] for c in range(CHANNELS)]
    ask_tokens = [vocab - 1 - CHANNELS * KEYS_PER_CHANNEL - c for c in range(CHANNELS)]
    embed = tensors["model.embed_tokens.weight"]
    for c in range(CHANNELS):
        low, high = head_dim // 2 - 1 - c, head_dim - 1 - c   # the pair (j, j + D/2) with the c-th slowest turn
        for name, rows in (("k_proj", [0]), ("q_proj", [0, head_dim])):
            for base in rows:
                tensors[p + name + ".weight"][base + low] = 0.0
                tensors[p + name + ".weight"][base + high] = 0.0
                tensors[p + name + ".bias"][base + low] = 0.0
                tensors[p + name + ".bias"][base + high] = 0.0
                tensors[p + name + ".weight"][base + high, c if name == "k_proj" else CHANNELS + c] = 1.7
        for i, token in enumerate(key_tokens[c]):
            embed[token] = 0.0
            embed[token, c] = 0.1
            embed[token, 2 * CHANNELS + c * KEYS_PER_CHANNEL + i] = 0.1  # each key token's value is its own
        embed[ask_tokens[c]] *= 0.25
        embed[ask_tokens[c], CHANNELS + c] = 0.1
    tensors = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    write_tensors(folder, raw, tensors)
    return raw, tensors, key_tokens, ask_tokens


@pytest.fixture(scope="module")
def long_case(tmp_path_factory):
    folder = tmp_path_factory.mktemp("long_32768")
    raw, tensors, key_tokens, ask_tokens = _planted_model(folder)
    plain_ids = raw["vocab_size"] - CHANNELS * (KEYS_PER_CHANNEL + 1)
    rng = random.Random(5)
    long_tokens = [rng.randrange(plain_ids) for _ in range(LONG)]
    for index, position in enumerate(KEY_POSITIONS):
        long_tokens[position] = key_tokens[index % CHANNELS][index // CHANNELS]
    portion = 2048
    ends = list(range(portion - 1, LONG - 32, portion))  # the last token of every portion asks
    for index, position in enumerate(ends):
        long_tokens[position] = ask_tokens[index % CHANNELS]
    for index, position in enumerate(range(LONG - 32, LONG)):  # and so does every single token at the end
        long_tokens[position] = ask_tokens[(index // 2) % CHANNELS] if index % 2 == 0 else rng.randrange(plain_ids)
    short_tokens = [rng.randrange(raw["vocab_size"]) for _ in range(90)]
    requests = {"long": long_tokens, "short": short_tokens}

    # the long prompt in portions of 2,048 tokens; its last 32 tokens one by one beside the short request, which
    # brings a portion first and single tokens then
    steps = []
    fed = 0
    while fed < LONG - 32:
        size = min(portion, LONG - 32 - fed)
        want = sorted({size - 1, rng.randrange(size), 0})
        steps.append({"step": len(steps), "entries": [{"id": "long", "tokens": long_tokens[fed: fed + size], "want": want}],
                      "end": []})
        fed += size
    short_fed = 0
    for index in range(32):
        size = 50 if index == 0 else 1
        entries = [{"id": "long", "tokens": [long_tokens[fed]], "want": [0]},
                   {"id": "short", "tokens": short_tokens[short_fed: short_fed + size], "want": [size - 1]}]
        fed += 1
        short_fed += size
        steps.append({"step": len(steps), "entries": entries, "end": ["long", "short"] if index == 31 else []})
    assert fed == LONG and short_fed <= len(short_tokens)
    requests["short"] = short_tokens[:short_fed]

    weights = {k: v.float() for k, v in tensors.items()}
    wanted: dict[str, list[int]] = {"long": [], "short": []}
    at = {"long": 0, "short": 0}
    for step in steps:
        for entry in step["entries"]:
            wanted[entry["id"]].extend(at[entry["id"]] + place for place in entry["want"])
            at[entry["id"]] += len(entry["tokens"])
    expected, rough = {}, {}
    for rid, tokens in requests.items():
        for out, dtype in ((expected, torch.float32), (rough, torch.bfloat16)):
            logits = plain_qwen2.forward(raw, weights, tokens, dtype=dtype, query_chunk=2048, rows=wanted[rid])
            out[rid] = torch.zeros((len(tokens), raw["vocab_size"]))
            out[rid][torch.tensor(wanted[rid])] = logits
    return folder, raw, requests, steps, expected, ask_tokens, weights, rough


def test_a_lost_key_would_show_at_32768_tokens(long_case):
    """The yardstick itself: without one planted key the plain logits of a row that asks for it move by far
    more than the tolerance of 16 bits."""
    _, raw, requests, _, expected, ask_tokens, weights, rough = long_case
    tokens = list(requests["long"][:4096])
    row = 4095
    assert tokens[row] in ask_tokens
    channel = ask_tokens.index(tokens[row])
    position = KEY_POSITIONS[channel]  # the channel's first key
    with_key = expected["long"][row]
    tokens[position] = 3
    without = plain_qwen2.forward(raw, weights, tokens, query_chunk=2048, rows=[row])[0]
    moved = float((with_key - without).abs().max())
    allowed = 1.5 * max(float((rough[rid] - expected[rid]).abs().max()) for rid in expected)
    print(f"logits move by {moved:.3f} when the key at {position} goes; bfloat16 may move them by {allowed:.3f}", flush=True)
    assert moved > 4 * allowed


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_32768_tokens_of_context(long_case, dtype, graph):
    """A prompt as long as the configuration allows, in portions of 2,048 tokens, and its last 32 tokens one
    by one beside a second request, eager and from captured graphs.  (The rows that ask for the planted keys
    have scores of 23, which 16-bit queries and keys move by a tenth: bfloat16 is held to what the plain
    implementation run in bfloat16 reaches, not to a fixed tolerance.)"""
    folder, raw, requests, steps, expected, _, _, rough = long_case
    page = 16
    pool = replay_util.max_live_tokens(steps, page=page)
    runner = make_runner(folder, dtype, pool, page, max_running=2, graph_decode=graph)
    print(f"32,768 tokens, {dtype}, graphs {graph}: {len(steps)} steps, pool {pool}", flush=True)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    if dtype == "float32":
        worst = replay_util.compare(rows, expected, every_position=False, rtol=2e-4, atol=1e-4)
        print(f"worst |diff| {worst:.3e}", flush=True)
    else:
        print("rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
              % replay_util.closer_than_plain_bfloat16(rows, expected, rough), flush=True)
    if graph:
        assert runner.graph_replays >= 30
    assert runner.cache.stats().pages_used == 0


# ---------------------------------------------------------------------------------------------------------
# decode steps of 64, 128 and 200 requests
# ---------------------------------------------------------------------------------------------------------

def _wide_decode(requests: dict[str, list[int]], tails: dict[str, int], per_step: int = 25) -> list[dict]:
    """Prompts whole, ``per_step`` requests to a step; then every live request brings one token a step until
    its tokens end, so that the steps narrow as the shorter tails run out."""
    steps = []
    names = list(requests)
    fed = {}
    for first in range(0, len(names), per_step):
        entries = []
        for rid in names[first: first + per_step]:
            head = len(requests[rid]) - tails[rid]
            entries.append({"id": rid, "tokens": requests[rid][:head], "want": [head - 1]})
            fed[rid] = head
        steps.append({"step": len(steps), "entries": entries, "end": []})
    while fed:
        entries, end = [], []
        for rid in list(fed):
            entries.append({"id": rid, "tokens": [requests[rid][fed[rid]]], "want": [0]})
            fed[rid] += 1
            if fed[rid] == len(requests[rid]):
                end.append(rid)
                del fed[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def _wide_case(raw, seed):
    rng = random.Random(seed)
    requests, tails = {}, {}
    for index in range(200):
        tail = 9 if index < 64 else 6 if index < 128 else 3
        rid = f"w{index}"
        requests[rid] = [rng.randrange(raw["vocab_size"]) for _ in range(rng.randint(2, 14) + tail)]
        tails[rid] = tail
    steps = _wide_decode(requests, tails)
    widths = sorted({len(step["entries"]) for step in steps if all(len(e["tokens"]) == 1 for e in step["entries"])})
    assert widths == [64, 128, 200]
    return requests, steps


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_64_to_200_requests_match_plain(tiny_folders, dtype, graph):
    """200 requests decode side by side, then 128, then 64 (Tiny-B): the buckets of 256, 128 and 64 rows."""
    folder, raw, tensors = tiny_folders["B"]
    requests, steps = _wide_case(raw, seed=41)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    runner = make_runner(folder, dtype, replay_util.max_live_tokens(steps, page=8), 8, max_running=200, graph_decode=graph)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    replay_util.compare(rows, {rid: expected[rid] for rid in rows}, every_position=False, **TOL[dtype])
    if dtype == "bfloat16":
        rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
        replay_util.closer_than_plain_bfloat16(rows, expected, rough)
    if graph:
        assert sorted(runner.graphs.buckets) == [64, 128, 256] and runner.graph_replays >= 9
    assert runner.cache.stats().pages_used == 0


@pytest.fixture(scope="module")
def wide_3b_case(tmp_path_factory):
    from cie_amd.workloads import SHAPES

    raw = dict(SHAPES["3b"], architectures=["Qwen2ForCausalLM"], num_hidden_layers=1, vocab_size=1031, eos_token_id=1030)
    folder, tensors = make_folder(tmp_path_factory.mktemp("wide_3b"), raw, seed=19, factor=1.5)
    requests, steps = _wide_case(raw, seed=43)
    weights = {k: v.float() for k, v in tensors.items()}
    expected = {rid: plain_qwen2.forward(raw, weights, tokens) for rid, tokens in requests.items()}
    # (at a width of 2,048 what bfloat16 costs is measured on the plain implementation, not assumed)
    rough = {rid: plain_qwen2.forward(raw, weights, tokens, dtype=torch.bfloat16) for rid, tokens in requests.items()}
    return folder, requests, steps, expected, rough


@pytest.mark.parametrize("graph", [False, True])
def test_decode_steps_of_64_to_200_requests_at_the_widths_of_the_3b_shape(wide_3b_case, graph):
    """The same steps with one layer of the 3B shape's widths (a short vocabulary), bfloat16: the products of
    64 to 256 rows that serving runs, against the plain implementation."""
    folder, requests, steps, expected, rough = wide_3b_case
    runner = make_runner(folder, "bfloat16", replay_util.max_live_tokens(steps, page=16), 16, max_running=200,
                         graph_decode=graph)
    rows = replay_util.by_position(steps, replay_util.drive_runner(runner, steps))
    print("rms %.3e worst %.3e, plain in bfloat16 %.3e %.3e"
          % replay_util.closer_than_plain_bfloat16(rows, expected, rough), flush=True)
    if graph:
        assert sorted(runner.graphs.buckets) == [64, 128, 256]
    assert runner.cache.stats().pages_used == 0


# ---------------------------------------------------------------------------------------------------------
# the smallest and the largest pages
# ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("page", [1, 2, 128, 256])
@pytest.mark.parametrize("name,seed", [("A", 3), ("B", 4), ("wide", 5)])
def test_random_traces_at_the_smallest_and_largest_pages(tiny_folders, tmp_path_factory, name, seed, page):
    """Pages of one and two tokens (every token on a page's edge) and of 128 and 256 (more than the blocks of
    keys the attention kernels step by), under traces drawn at random, in both precisions, eager and captured;
    ``wide`` has heads of 128 dimensions, the size whose prompt portions take the forms of four and eight waves."""
    rng = random.Random(100 * seed + page)
    if name == "wide":
        raw = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", hidden_size=128, num_hidden_layers=2,
                   num_attention_heads=4, num_key_value_heads=2, head_dim=128, intermediate_size=192, vocab_size=331,
                   rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=1200, tie_word_embeddings=True,
                   attention_bias=True, use_sliding_window=False, eos_token_id=1)
        folder, tensors = make_folder(tmp_path_factory.mktemp(f"pages_{page}"), raw, seed=seed, factor=4.0)
    else:
        folder, raw, tensors = tiny_folders[name]
    longest = raw["max_position_embeddings"]
    lengths = [rng.randint(1, longest) for _ in range(rng.randint(2, 5))] + [longest]
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
