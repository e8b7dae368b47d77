"""GPU: the whole engine through its entry points: greedy generation against the
plain implementation, long decoding, the first tokens of a sequence, temperature
sampling, cache pressure with recompute preemption, prefix reuse, random requests
through a small pool against each request alone, the command line."""

from __future__ import annotations

import json
import subprocess
import sys

import pytest
import torch

import plain_qwen2 as plain
from conftest import ROOT, TINY, random_tokens

pytestmark = pytest.mark.gpu


def float_weights(tensors):
    return {k: v.float() for k, v in tensors.items()}


def make_engine(folder, dtype="float32", **options):
    from cie_amd import Engine

    defaults = dict(page_size=8, kv_tokens=1024, max_running=8, prefill_chunk=16, token_budget=48,
                    prefix_cache_pages=0)
    defaults.update(options)
    return Engine(folder, dtype=dtype, **defaults)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(tiny_folders, name):
    """Engine.generate in float32: chunked prefill mixed with decoding of other
    requests yields exactly the plain implementation's greedy tokens."""
    from cie_amd import GenerationConfig

    folder, raw, tensors = tiny_folders[name]
    lengths = [5, 17, 33] if name == "A" else [1, 9, 40, 64, 100]
    prompts = [random_tokens(n, raw["vocab_size"], 200 + i) for i, n in enumerate(lengths)]
    engine = make_engine(folder, page_size=16 if name == "A" else 8)
    results = engine.generate(prompts, GenerationConfig(max_output_tokens=8, eos_token_id=None))
    weights = float_weights(tensors)
    for prompt, result in zip(prompts, results):
        expected = plain.generate_greedy(raw, weights, prompt, 8)
        assert result.token_ids == expected, f"prompt of {len(prompt)} tokens"
        assert (result.input_tokens, result.output_tokens) == (len(prompt), 8)
        assert result.finish_reason == "max_output_tokens_reached" and result.ttft_ms is not None
    metrics = engine.snapshot_metrics()
    assert metrics["requests"]["completed_total"] == len(prompts) and metrics["kv_cache"]["pages_used"] == 0
    assert metrics["runner"]["max_forward_request_count"] > 1, "requests shared forwards"
    assert metrics["tokens"]["output_total"] == 8 * len(prompts)


def test_eos_stops_generation(tiny_folders):
    from cie_amd import GenerationConfig

    folder, raw, tensors = tiny_folders["A"]
    prompt = random_tokens(12, raw["vocab_size"], 300)
    expected = plain.generate_greedy(raw, float_weights(tensors), prompt, 6)
    engine = make_engine(folder)
    result = engine.generate([prompt], GenerationConfig(max_output_tokens=6, eos_token_id=expected[2]))[0]
    stop = expected.index(expected[2])
    assert result.token_ids == expected[: stop + 1] and result.finish_reason == "eos_token_reached"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(tiny_folders, dtype):
    """A prompt of one token, then 150 decode steps: every step's logits against
    the plain implementation run on the whole generated sequence (teacher forced
    on the engine's own tokens); positions 0..7 are checked on their own."""
    from cie_amd.engine.runner import StepEntry

    folder, raw, tensors = tiny_folders["B"]
    engine = make_engine(folder, dtype=dtype, kv_tokens=160, max_model_len=160)
    runner = engine.runner
    runner.cache.admit("long")
    tokens = [3]
    rows = []
    for step in range(150):
        logits = runner.run([StepEntry("long", [tokens[-1]], step, [0])])
        rows.append(logits[0].float().cpu())
        tokens.append(int(logits[0].argmax()))
    expected = plain.forward(raw, float_weights(tensors), tokens[:-1])
    got = torch.stack(rows)
    tol = dict(rtol=1e-4, atol=2e-5) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(got[:8], expected[:8], **tol)
    torch.testing.assert_close(got, expected, **tol)
    if dtype == "float32":
        assert tokens[1:] == [int(r.argmax()) for r in expected]
    runner.cache.release("long")
    assert runner.cache.stats().pages_used == 0


def test_temperature_sampling_is_seeded_and_independent_of_the_batch(tiny_folders):
    from cie_amd import GenerationConfig

    folder, raw, _ = tiny_folders["B"]
    prompts = [random_tokens(n, raw["vocab_size"], 400 + n) for n in (9, 40, 64)]
    gen = [GenerationConfig(max_output_tokens=12, temperature=0.8, eos_token_id=None, seed=50 + i) for i in range(3)]
    together = make_engine(folder, token_budget=48).generate(prompts, gen)
    alone = [make_engine(folder, token_budget=7, prefill_chunk=5).generate([p], [g])[0] for p, g in zip(prompts, gen)]
    assert [r.token_ids for r in together] == [r.token_ids for r in alone]
    other_seed = make_engine(folder).generate(prompts[:1], GenerationConfig(max_output_tokens=12, temperature=0.8, seed=7))
    assert other_seed[0].token_ids != together[0].token_ids
    greedy = make_engine(folder).generate(prompts[:1], GenerationConfig(max_output_tokens=12, eos_token_id=None))
    assert greedy[0].token_ids != together[0].token_ids  # the draws are not all argmax


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_tokens_are_the_inverse_cdf_of_the_plain_logits(tiny_folders, dtype):
    """Not engine against engine: the expected ids come from the plain model's logits, the uniform number
    the sampler documents for (seed, token index), and a plain inverse CDF."""
    import replay_util
    from cie_amd import GenerationConfig
    from cie_amd.sampling.sampler import uniform_for

    folder, raw, tensors = tiny_folders["A"]
    weights = float_weights(tensors)
    prompts = [random_tokens(n, raw["vocab_size"], 450 + n) for n in (6, 21, 37)]
    gens = [GenerationConfig(max_output_tokens=16, temperature=t, eos_token_id=None, seed=90 + i)
            for i, t in enumerate((0.7, 1.0, 1.6))]
    results = make_engine(folder, dtype=dtype, page_size=16, token_budget=24).generate(prompts, gens)
    slack = 1e-4 if dtype == "float32" else 2e-2  # (of the unit interval: what a logit's rounding moves a boundary by)
    boundary = 0
    for prompt, gen, result in zip(prompts, gens, results):
        uniforms = [uniform_for(gen.seed, 0, i) for i in range(16)]
        boundary += replay_util.drawn_tokens_follow_plain(
            lambda tokens: plain.forward(raw, weights, tokens), prompt, result.token_ids, gen.temperature, uniforms, slack)
        assert len(set(result.token_ids)) > 4, "draws, not one token over and over"
    assert boundary <= (0 if dtype == "float32" else 6)


def test_pressure_preempts_and_recomputes_to_the_same_tokens(tiny_folders):
    """A pool too small for two requests at once (reference
    tests/remote_ragged_gpu_tests.py:294-332): preemptions > 0, recomputed tokens
    > 0, outputs identical to the unpressured run, allocator drained."""
    from cie_amd import GenerationConfig

    folder, raw, _ = tiny_folders["A"]
    prompts = [random_tokens(56, raw["vocab_size"], 500 + i) for i in range(2)]
    gen = GenerationConfig(max_output_tokens=12, eos_token_id=None)
    roomy = make_engine(folder, page_size=16, kv_tokens=512).generate(prompts, gen)
    tight = make_engine(folder, page_size=16, kv_tokens=128)  # 8 pages; each request ends at 68 tokens = 5 pages
    results = tight.generate(prompts, gen)
    assert [r.token_ids for r in results] == [r.token_ids for r in roomy]
    metrics = tight.snapshot_metrics()
    assert metrics["requests"]["preempted_total"] > 0 and metrics["tokens"]["recomputed_total"] > 0
    assert metrics["kv_cache"]["pages_used"] == 0
    tight.runner.cache.assert_invariants()


def test_prefix_reuse_keeps_tokens_and_saves_work(tiny_folders):
    """reference tests/remote_ragged_gpu_tests.py:335-377: the same prompt twice
    gives identical tokens, the warm run feeds at least a page less, hits >= 1,
    request pages 0 and prefix pages > 0 afterwards.  Beyond it: a prompt that
    shares only the first pages and then differs also hits."""
    from cie_amd import GenerationConfig

    folder, raw, tensors = tiny_folders["A"]
    prompt = random_tokens(45, raw["vocab_size"], 600)
    sibling = prompt[:32] + random_tokens(9, raw["vocab_size"], 601)
    gen = GenerationConfig(max_output_tokens=6, eos_token_id=None)
    engine = make_engine(folder, page_size=16, prefix_cache_pages=8)
    cold = engine.generate([prompt], gen)[0]
    cold_work = engine.snapshot_metrics()["tokens"]["input_total"]
    warm = engine.generate([prompt], gen)[0]
    warm_work = engine.snapshot_metrics()["tokens"]["input_total"] - cold_work
    assert warm.token_ids == cold.token_ids
    assert warm_work + 16 <= cold_work
    third = engine.generate([sibling], gen)[0]
    assert third.token_ids == plain.generate_greedy(raw, float_weights(tensors), sibling, 6)
    cache = engine.snapshot_metrics()["kv_cache"]
    assert cache["prefix_cache_hits"] >= 2 and cache["request_pages_used"] == 0 and cache["prefix_pages_used"] > 0
    engine.runner.cache.assert_invariants()


def test_prefix_is_shared_with_a_request_that_arrives_while_the_first_still_decodes(tiny_folders):
    """The first request's prompt pages are offered to the index when its prompt is
    done, not when it ends: a sibling submitted during its decoding takes them over,
    both go on writing behind the shared pages, and both match the plain model."""
    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    folder, raw, tensors = tiny_folders["A"]
    prompt = random_tokens(45, raw["vocab_size"], 610)
    sibling = prompt[:32] + random_tokens(9, raw["vocab_size"], 611)
    gen = GenerationConfig(max_output_tokens=12, eos_token_id=None)
    engine = make_engine(folder, page_size=16, prefix_cache_pages=8)
    first = engine.submit(prompt, gen)
    while len(first.output) < 3:
        engine.step()
    assert first.state is RequestState.DECODING
    second = engine.submit(sibling, gen)
    while engine.has_work():
        engine.step()
    weights = float_weights(tensors)
    assert engine.result_of(first).token_ids == plain.generate_greedy(raw, weights, prompt, 12)
    assert engine.result_of(second).token_ids == plain.generate_greedy(raw, weights, sibling, 12)
    cache = engine.snapshot_metrics()["kv_cache"]
    assert cache["prefix_cache_hits"] == 1 and cache["request_pages_used"] == 0
    # tokens run through the model: both prompts less the 32 shared tokens, plus the decoded tokens fed back
    assert engine.snapshot_metrics()["tokens"]["input_total"] <= len(prompt) + len(sibling) - 32 + 2 * 12
    engine.runner.cache.assert_invariants()


def test_bfloat16_under_pressure_with_shared_prefixes_follows_the_plain_model(tiny_folders):
    """bfloat16 with everything on at once: a pool that forces preemption, prompts that share their first
    pages, captured decode steps started ahead of their tokens.  Every request's tokens follow the plain
    model, near-ties that bfloat16 may turn aside."""
    import replay_util
    from cie_amd import GenerationConfig

    folder, raw, tensors = tiny_folders["A"]
    weights = float_weights(tensors)
    shared = random_tokens(32, raw["vocab_size"], 650)
    prompts = [shared + random_tokens(8 + 3 * i, raw["vocab_size"], 651 + i) for i in range(4)]
    gen = GenerationConfig(max_output_tokens=14, eos_token_id=None)
    tight = make_engine(folder, dtype="bfloat16", page_size=16, kv_tokens=160, max_running=4, prefix_cache_pages=4,
                        token_budget=32, prefill_chunk=16, admit_within_pool=False, max_model_len=128)
    results = tight.generate(prompts, gen)
    metrics = tight.snapshot_metrics()
    assert metrics["requests"]["preempted_total"] > 0 and metrics["kv_cache"]["prefix_cache_hits"] > 0
    assert metrics["runner"]["graph_replays"] > 0 and metrics["kv_cache"]["request_pages_used"] == 0
    tight.runner.cache.assert_invariants()
    turned = 0
    for prompt, result in zip(prompts, results):
        assert len(result.token_ids) == 14
        turned += replay_util.greedy_tokens_follow_plain(
            lambda tokens: plain.forward(raw, weights, tokens), prompt, result.token_ids,
            lambda tokens: plain.forward(raw, weights, tokens, dtype=torch.bfloat16))
    assert turned <= 6


def test_random_requests_through_a_small_pool_equal_each_request_alone(tiny_folders):
    """Forty random requests (shared prefixes, greedy and seeded temperature sampling, end
    tokens) arrive a few per step at an engine whose pool holds one and a half full sequences: with
    preemption, prefix sharing, captured decode steps and tokens fed back on the device, every
    request ends with the tokens it gets when it runs alone, and the pool drains."""
    import random

    from cie_amd import GenerationConfig

    folder, raw, _ = tiny_folders["B"]
    rng = random.Random(3)
    limit, vocab = raw["max_position_embeddings"], raw["vocab_size"]
    prefix = [rng.randrange(vocab) for _ in range(40)]
    requests = []
    for _ in range(40):
        count = rng.randint(2, limit // 2)
        prompt = prefix[: rng.randint(0, min(40, count - 1))] if rng.random() < 0.5 else []
        prompt = prompt + [rng.randrange(vocab) for _ in range(count - len(prompt))]
        gen = GenerationConfig(max_output_tokens=rng.randint(1, min(40, limit - count - 1)),
                               eos_token_id=rng.choice([None, None, rng.randrange(vocab)]),
                               temperature=rng.choice([0.0, 0.0, 0.7, 1.3]), seed=rng.randrange(1000))
        requests.append((prompt, gen))
    busy = make_engine(folder, page_size=8, kv_tokens=3 * limit // 2, max_running=8, max_queue_size=64,
                       max_model_len=limit, max_output_tokens=64, token_budget=64, prefill_chunk=7,
                       prefix_cache_pages=16, admit_within_pool=False)
    handles, pending, steps = [], list(requests), 0
    while pending or busy.has_work():
        for _ in range(rng.randint(0, 3)):
            if pending:
                handles.append(busy.submit(*pending.pop(0)))
        busy.step()
        steps += 1
        assert steps < 4000, "the engine does not drain"
    results = [busy.result_of(handle) for handle in handles]
    metrics = busy.snapshot_metrics()
    assert metrics["requests"]["preempted_total"] > 0 and metrics["kv_cache"]["prefix_cache_hits"] > 0
    assert metrics["kv_cache"]["request_pages_used"] == 0
    # (portions of 7 tokens beside the same few decoding requests: shapes of steps that come again and are captured)
    assert metrics["runner"]["mixed_graph_replays"] > 0 and metrics["runner"]["graph_replays"] > 0
    busy.runner.cache.assert_invariants()
    alone = make_engine(folder, page_size=16, kv_tokens=2 * limit, max_running=1, max_model_len=limit,
                        max_output_tokens=64, graph_decode=False, async_decode=False)
    for (prompt, gen), got in zip(requests, results):
        want = alone.generate([prompt], gen)[0]
        assert (want.token_ids, want.finish_reason) == (got.token_ids, got.finish_reason), (len(prompt), gen)


def test_warm_up_captures_every_decode_bucket_once(tiny_folders):
    from cie_amd import GenerationConfig

    folder, raw, tensors = tiny_folders["B"]
    engine = make_engine(folder, dtype="bfloat16", max_running=6, graph_decode=True)
    assert engine.warm_up() == 4  # buckets of 1, 2, 4 and 8 rows for up to 6 requests
    assert engine.warm_up() == 0
    prompts = [random_tokens(n, raw["vocab_size"], 700 + n) for n in (3, 9, 20, 33, 40)]
    results = engine.generate(prompts, GenerationConfig(max_output_tokens=10, eos_token_id=None))
    runner = engine.snapshot_metrics()["runner"]
    assert runner["graph_captures"] == 4 and runner["graph_replays"] >= 9
    import replay_util

    weights = float_weights(tensors)
    turned = 0
    for prompt, result in zip(prompts, results):
        # every token is the plain model's after the same context, or a near-tie that bfloat16 may turn
        assert len(result.token_ids) == 10
        turned += replay_util.greedy_tokens_follow_plain(
            lambda tokens: plain.forward(raw, weights, tokens), prompt, result.token_ids,
            lambda tokens: plain.forward(raw, weights, tokens, dtype=torch.bfloat16))
    assert turned <= 5, "most of the 50 tokens are the plain model's own"


def test_step_refuses_what_it_cannot_run(tiny_folders):
    from cie_amd.cache import CacheCapacityFull
    from cie_amd.engine.runner import StepEntry

    folder, raw, _ = tiny_folders["A"]
    runner = make_engine(folder, page_size=16, kv_tokens=32, max_model_len=32).runner
    runner.cache.admit("a"), runner.cache.admit("b")
    with pytest.raises(ValueError, match="outside the vocabulary"):
        runner.run([StepEntry("a", [raw["vocab_size"]], 0, [0])])
    with pytest.raises(ValueError, match="continues at 3"):
        runner.run([StepEntry("a", [1], 3, [0])])
    with pytest.raises(ValueError, match="twice"):
        runner.run([StepEntry("a", [1], 0, []), StepEntry("a", [2], 1, [])])
    with pytest.raises(ValueError, match="wanted place"):
        runner.run([StepEntry("a", [1, 2], 0, [2])])
    runner.run([StepEntry("a", list(range(20)), 0, [])])
    with pytest.raises(CacheCapacityFull):
        runner.run([StepEntry("b", list(range(20)), 0, [])])  # 2 pages needed, none free
    assert runner.cache.length("a") == 20 and runner.cache.length("b") == 0
    assert runner.cache.block_table(0, "b") == []  # nothing changed


def test_command_line_generates(tiny_folders, tmp_path):
    folder, raw, tensors = tiny_folders["A"]
    prompt = [7, 8, 9, 10, 11]
    expected = plain.generate_greedy(raw, float_weights(tensors), prompt, 5)
    done = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "cie"), "generate", "--token-ids", " ".join(map(str, prompt)),
         "--model", str(folder), "--max-output-tokens", "5", "--dtype", "fp32", "--no-stream", "--ignore-eos",
         "--max-model-len", "64", "--kv-tokens", "256"],
        capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split() == [str(t) for t in expected]
    config_path = tmp_path / "config.json"
    config_path.write_text(json.dumps(TINY["B"]))
    out_dir = tmp_path / "model"
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "cie"), "init-model", "--config", str(config_path),
                           "--out", str(out_dir), "--seed", "4"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and (out_dir / "model.safetensors").is_file() and (out_dir / "config.json").is_file()
    done = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "cie"), "generate", "--token-ids", "1,2,3", "--model", str(out_dir),
         "--max-output-tokens", "4", "--temperature", "0.8", "--seed", "3", "--metrics", "--max-model-len", "64",
         "--kv-pages", "12", "--page-size", "8"],
        capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert '"completed_total": 1' in done.stdout and '"pages_total": 12' in done.stdout
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "cie"), "generate", "--token-ids", "1", "--model", str(out_dir),
                           "--kv-pages", "12", "--kv-tokens", "96"], capture_output=True, text=True, timeout=300)
    assert done.returncode != 0 and "give one" in done.stderr


@pytest.mark.parametrize("from_folder", [False, True])
def test_loading_needs_the_models_own_size_of_device_memory_not_twice(tmp_path, from_folder):
    """A model's tensors are made one by one while it binds them (its own forms of some are copies: q/k/v as one
    matrix, gate and up as one), so loading peaks at the model's size plus a layer's tensors."""
    from cie_amd.config import config_from_dict
    from cie_amd.engine.loading import load_model, random_model
    from cie_amd.weights import write_model_folder

    raw = dict(TINY["A"], hidden_size=512, intermediate_size=2048, num_attention_heads=8, num_key_value_heads=2,
               head_dim=64, num_hidden_layers=12, vocab_size=1024)
    config = config_from_dict(raw)
    if from_folder:
        write_model_folder(tmp_path, config, seed=2)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    model = load_model(tmp_path, "bfloat16")[0] if from_folder else random_model(config, 2, draw_device="cuda")
    held = torch.cuda.memory_allocated() - before
    peak = torch.cuda.max_memory_allocated() - before
    per_layer = held / raw["num_hidden_layers"]
    assert held > 80e6  # (about 90 MB: the check below is about something)
    assert peak < held + 4 * per_layer, (held, peak)
    del model


def test_the_pool_is_sized_by_what_the_requests_can_use_or_by_the_memory_that_is_free(tiny_folders):
    """Without a size the pool takes a fraction of the free device memory, but never more pages than max_running
    requests of max_model_len tokens and the prefix index can use; a size in bytes or tokens is taken as given."""
    from cie_amd import Engine

    folder, raw, _ = tiny_folders["A"]
    engine = Engine(folder, dtype="bfloat16", max_running=3, max_model_len=100, page_size=16, prefix_cache_pages=5)
    assert engine.runner.cache.stats().pages_total == 3 * 7 + 5  # 7 pages a request: 100 tokens
    head_width = engine.runner.model.cache_needs()[0].head_dim  # (heads of 16 lie in the cache as the heads of 32 the kernels take)
    assert head_width == 32
    per_token = 2 * raw["num_hidden_layers"] * raw["num_key_value_heads"] * head_width * 2  # keys and values, bfloat16
    engine = Engine(folder, dtype="bfloat16", max_running=3, max_model_len=100, page_size=16, kv_cache_bytes=40 * per_token)
    assert engine.runner.cache.stats().pages_total == 2  # 40 tokens' worth: two whole pages
    engine = Engine(folder, dtype="bfloat16", max_running=3, max_model_len=100, page_size=16, kv_tokens=64)
    assert engine.runner.cache.stats().pages_total == 4


def test_a_serving_workload_runs_and_its_tokens_do_not_depend_on_the_batch():
    """``cie workload`` on a profile made small (one layer of the smallest shape, six requests, float32): the record's
    fields, and the first requests run once more, alone, give the same tokens (``run_profile`` raises if not)."""
    from dataclasses import replace

    from cie_amd.workloads import PROFILES, run_profile

    profile = replace(PROFILES["mixed"], requests=6)
    record = run_profile(profile, layers=1, dtype="float32", shape="0.5b", verify=3)
    assert record["verified"] == {"requests": 3, "same_tokens_alone": 3}
    assert (record["workload"], record["shape"], record["layers"], record["layers_full"], record["requests"]) == \
        ("mixed", "0.5b", 1, 24, 6)
    assert record["output_tokens"] > 0 and record["input_tokens"] > 0 and record["elapsed_s"] > 0
    assert record["output_tokens_per_s"] == pytest.approx(record["output_tokens"] / record["elapsed_s"], rel=0.01)
    for key in ("ttft_ms", "itl_ms", "e2e_ms"):
        assert record[key]["p50"] <= record[key]["p95"]
    assert record["preempted"] == 0 and "synthetic" in record["data"]


def test_ceilings_reports_what_the_gpu_reaches():
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "cie"), "ceilings"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    record = json.loads(done.stdout.strip().splitlines()[-1])
    # what this kind of box has reached before (one MI355X, the record under profiles/), give or take 30 %: a
    # figure outside of that is a measurement gone wrong (a timer around the wrong thing, a product that is
    # not the one named), or a box in another state than any seen so far
    seen_before = {"copy_1GiB_GBps": 5159.4, "read_1GiB_library_mv_GBps": 5402.1, "read_1GiB_few_row_product_GBps": 5549.7,
                   "read_45MB_few_row_product_GBps": 4277.2, "bf16_8192_cubed_library_TFLOPs": 1420.6,
                   "bf16_8192_cubed_library_tuned_TFLOPs": 1578.3}
    for key, before in seen_before.items():
        assert 0.7 * before <= record[key] <= 1.3 * before, (key, record[key], before)
    assert record["bf16_8192_cubed_library_tuned_TFLOPs"] >= 0.97 * record["bf16_8192_cubed_library_TFLOPs"]


def test_text_prompts_go_through_the_folders_tokenizer(tiny_folders, tmp_path):
    """A prompt given as text is cut by the ``tokenizer.json`` of the model folder and the result comes back as text
    too (a word-level tokenizer made here, over the tiny model's 256 ids); without that file text is refused with
    a message and token ids still work."""
    import shutil

    from tokenizers import Tokenizer, decoders, models, pre_tokenizers

    from cie_amd import Engine, GenerationConfig

    folder, raw, tensors = tiny_folders["A"]
    with_words = tmp_path / "with_tokenizer"
    shutil.copytree(folder, with_words)
    tokenizer = Tokenizer(models.WordLevel({f"w{i}": i for i in range(raw["vocab_size"])}, unk_token="w0"))
    tokenizer.pre_tokenizer = pre_tokenizers.Whitespace()
    tokenizer.decoder = decoders.WordPiece(prefix="##")
    tokenizer.save(str(with_words / "tokenizer.json"))
    prompt = [7, 8, 9, 10, 11]
    expected = plain.generate_greedy(raw, float_weights(tensors), prompt, 5)
    engine = make_engine(with_words)
    gen = GenerationConfig(max_output_tokens=5, eos_token_id=None)
    result = engine.generate(["w7 w8 w9 w10 w11"], gen)[0]
    assert result.token_ids == expected and result.text == " ".join(f"w{t}" for t in expected)
    done = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "cie"), "generate", "w7 w8 w9 w10 w11", "--model", str(with_words),
         "--max-output-tokens", "5", "--dtype", "fp32", "--no-stream", "--ignore-eos", "--max-model-len", "64"],
        capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.split() == [f"w{t}" for t in expected]
    bare = make_engine(folder)
    with pytest.raises(ValueError, match="tokenizer.json"):
        bare.generate(["w7 w8"], gen)
    assert bare.generate([prompt], gen)[0].token_ids == expected


def test_command_line_metrics_prints_the_counters_of_a_run(tiny_folders):
    folder, _, _ = tiny_folders["B"]
    done = subprocess.run([sys.executable, str(ROOT / "bin" / "cie"), "metrics", "--model", str(folder), "--token-ids", "3 4 5",
                           "--max-output-tokens", "6", "--max-model-len", "64"], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    counters = json.loads(done.stdout)
    assert counters["requests"]["completed_total"] == 1 and counters["tokens"]["output_total"] <= 6
    assert counters["kv_cache"]["pages_used"] == counters["kv_cache"]["prefix_pages_used"]


def test_generation_with_profiler_ranges_switched_on(tiny_folders):
    """``ENGINE_NVTX=1`` puts named ranges around the phases of every iteration (torch emits them as roctx ranges):
    the same tokens come out."""
    import os

    folder, raw, tensors = tiny_folders["A"]
    prompt = [7, 8, 9, 10, 11]
    expected = plain.generate_greedy(raw, float_weights(tensors), prompt, 5)
    code = ("import sys; sys.path.insert(0, %r); import cie_amd\n"
            "from cie_amd import Engine, GenerationConfig, profiling\n"
            "assert profiling.trace_range('a') is not profiling.trace_range('b'), 'ranges are off'\n"
            "engine = Engine(%r, dtype='float32', kv_tokens=256, max_model_len=64)\n"
            "print(engine.generate([%r], GenerationConfig(max_output_tokens=5, eos_token_id=None))[0].token_ids)\n"
            ) % (str(ROOT), str(folder), prompt)
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300,
                          env={**os.environ, "ENGINE_NVTX": "1"})
    assert done.returncode == 0, done.stderr[-2000:]
    assert done.stdout.strip().splitlines()[-1] == str(expected)
