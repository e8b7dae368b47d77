"""Offline serving workloads: a set of requests run to completion through the
scheduler, with wall-clock throughput and latency percentiles.

Profiles follow the reference's offline benchmark (benchmarks/workloads.json:
``decode``, ``mixed``, ``fragmentation``; protocol of benchmarks/run.py:205-207,
241-256: fresh engine, all requests submitted at once, output tokens per
wall-clock second, TTFT / ITL percentiles from the engine's own metrics).  The
reference builds prompts from a word bank through a tokenizer; here prompts are
seeded uniform-random token ids of the stated lengths and weights are random,
EOS is ignored.  Two larger profiles exercise what the small ones do not: many
live requests with chunked prompts beside decoding ones, and long prompts with a
common prefix in a pool too small for all of them (prefix reuse; admission that
waits for room, or preemption and recomputation where all are admitted at once).
"""

from __future__ import annotations

import json
import random
import time
from dataclasses import dataclass, field, replace
from typing import Any

# Model shapes of the Qwen2.5 family (their config.json values); weights are random.
_COMMON = dict(model_type="qwen2", rope_theta=1e6, attention_bias=True, use_sliding_window=False,
               max_position_embeddings=32768, eos_token_id=151643)
SHAPES: dict[str, dict[str, Any]] = {
    "0.5b": dict(_COMMON, hidden_size=896, num_hidden_layers=24, num_attention_heads=14, num_key_value_heads=2,
                 intermediate_size=4864, vocab_size=151936, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "3b": dict(_COMMON, hidden_size=2048, num_hidden_layers=36, num_attention_heads=16, num_key_value_heads=2,
               intermediate_size=11008, vocab_size=151936, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "7b": dict(_COMMON, hidden_size=3584, num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4,
               intermediate_size=18944, vocab_size=152064, rms_norm_eps=1e-6, tie_word_embeddings=False),
    "14b": dict(_COMMON, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=13824, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
    # the family's two largest: 65 and 145 GB of bf16 weights, for one GPU's 288 GB
    "32b": dict(_COMMON, hidden_size=5120, num_hidden_layers=64, num_attention_heads=40, num_key_value_heads=8,
                intermediate_size=27648, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "72b": dict(_COMMON, hidden_size=8192, num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8,
                intermediate_size=29568, vocab_size=152064, rms_norm_eps=1e-5, tie_word_embeddings=False),
}


@dataclass(frozen=True)
class Profile:
    """``requests`` requests; prompt and output lengths uniform in their ranges;
    the first ``shared_prefix`` prompt tokens are the same for all requests.
    ``pool_fraction`` < 1 sizes the cache for that share of what all requests
    would hold at their ends, which forces preemption."""

    name: str
    shape: str
    requests: int
    prompt_tokens: tuple[int, int]
    output_tokens: tuple[int, int]
    shared_prefix: int = 0
    token_budget: int = 2048
    prefill_chunk: int = 512
    pool_fraction: float = 1.0
    lead_requests: int = 0  # submitted first; the others arrive when these have their first token
    purpose: str = ""
    engine_options: dict[str, Any] = field(default_factory=dict)


PROFILES: dict[str, Profile] = {p.name: p for p in (
    # benchmarks/workloads.json: profiles.decode / mixed / fragmentation
    Profile("decode", "3b", 8, (28, 36), (128, 128), purpose="decode throughput at fixed concurrency"),
    Profile("mixed", "3b", 16, (16, 512), (16, 128), purpose="continuous admission under heterogeneous load"),
    Profile("fragmentation", "3b", 16, (30, 34), (8, 256), purpose="cache use across short and long generations"),
    Profile("mixed-7b", "7b", 64, (128, 4096), (256, 256), token_budget=2048,
            purpose="64 live requests: prompt portions under a 2,048-token budget beside decoding requests"),
    Profile("prefix-14b", "14b", 32, (8192, 8192), (128, 128), shared_prefix=2048, pool_fraction=0.6, lead_requests=1,
            purpose="long prompts with a common 2,048-token prefix in a pool too small for all: prefix reuse, and "
                    "admission that waits for room"),
    Profile("pressure-14b", "14b", 32, (8192, 8192), (128, 128), shared_prefix=2048, pool_fraction=0.6, lead_requests=1,
            engine_options={"admit_within_pool": False},
            purpose="the same, all admitted at once as the reference admits: preemption and recomputation"),
)}


def make_requests(profile: Profile, vocab_size: int, seed: int) -> list[tuple[list[int], int]]:
    rng = random.Random(seed)
    prefix = [rng.randrange(vocab_size) for _ in range(profile.shared_prefix)]
    out = []
    for _ in range(profile.requests):
        length = rng.randint(*profile.prompt_tokens)
        own = max(length - len(prefix), 1)
        prompt = prefix[: length - own] + [rng.randrange(vocab_size) for _ in range(own)]
        out.append((prompt, rng.randint(*profile.output_tokens)))
    return out


def run_profile(profile: Profile, *, layers: int | None = None, dtype: str = "bfloat16", seed: int = 0,
                page_size: int = 16, shape: str | None = None, verify: int = 0) -> dict[str, Any]:
    """Run the profile on a fresh engine with random weights; returns the record that
    ``cie workload`` prints.  ``layers`` runs fewer layers than the shape has (the
    record names both numbers)."""
    import torch

    from . import Engine, GenerationConfig
    from .config import config_from_dict

    raw = dict(SHAPES[shape or profile.shape], architectures=["Qwen2ForCausalLM"])
    layers_full = raw["num_hidden_layers"]
    if layers is not None:
        raw["num_hidden_layers"] = layers
    config = config_from_dict(raw)
    requests = make_requests(profile, config.vocab_size, seed)
    longest = max(len(p) + n for p, n in requests)
    held = sum(-(-(len(p) + n) // page_size) * page_size for p, n in requests)
    kv_tokens = max(int(held * profile.pool_fraction), -(-longest // page_size) * page_size) + 4 * page_size
    prefix_pages = 2 * (-(-profile.shared_prefix // page_size)) if profile.shared_prefix else 0
    options = dict(
        dtype=dtype, page_size=page_size, kv_tokens=kv_tokens, max_running=profile.requests,
        max_queue_size=profile.requests + 1, max_model_len=longest + page_size, max_output_tokens=longest,
        token_budget=profile.token_budget, prefill_chunk=profile.prefill_chunk, prefix_cache_pages=prefix_pages,
    )
    options.update(profile.engine_options)
    engine = Engine(config=config, seed=seed, draw_device="cuda", **options)

    # warm-up outside the clock: decode graphs of all bucket sizes, and one short generation
    engine.warm_up()
    # (prompts long enough to go through the library's matrix products, which set themselves up at first use)
    warm = [engine.submit(list(range(1, 49)), GenerationConfig(max_output_tokens=4, eos_token_id=None)) for _ in range(2)]
    while engine.has_work():
        engine.step()
    assert all(r.is_final for r in warm)
    engine.metrics.reset()
    torch.cuda.synchronize()

    start = time.perf_counter()
    def submit(batch):
        return [engine.submit(prompt, GenerationConfig(max_output_tokens=n, eos_token_id=None)) for prompt, n in batch]

    steps = 0
    handles = submit(requests[: profile.lead_requests])
    while any(len(h.output) == 0 and not h.is_final for h in handles):
        engine.step()
        steps += 1
    handles += submit(requests[profile.lead_requests:])
    while engine.has_work():
        engine.step()
        steps += 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start

    results = [engine.result_of(h) for h in handles]
    snapshot = engine.snapshot_metrics()
    verified = None
    if verify:
        # each of the first requests once more, alone: in float32 every kernel gives a row the same result
        # whatever else is in the batch and however the prompt was cut, so the tokens must be the same
        engine.runner.cache.clear_prefix_index()
        same = 0
        for (prompt, n), result in list(zip(requests, results))[:verify]:
            alone = engine.generate([prompt], GenerationConfig(max_output_tokens=n, eos_token_id=None))[0]
            same += alone.token_ids == result.token_ids
        verified = {"requests": min(verify, len(requests)), "same_tokens_alone": same}
        if dtype == "float32" and same != verified["requests"]:
            raise AssertionError(f"float32 tokens depend on the batch: {verified}")
    output_tokens = sum(r.output_tokens for r in results)
    input_tokens = sum(r.input_tokens for r in results)
    assert all(r.output_tokens == n for r, (_, n) in zip(results, requests))
    return {
        "workload": profile.name, "purpose": profile.purpose, "shape": shape or profile.shape,
        "layers": config.num_hidden_layers, "layers_full": layers_full, "dtype": dtype,
        "requests": profile.requests, "input_tokens": input_tokens, "output_tokens": output_tokens,
        "kv_tokens": kv_tokens, "elapsed_s": round(elapsed, 4), "scheduler_steps": steps,
        "output_tokens_per_s": round(output_tokens / elapsed, 1),
        "total_tokens_per_s": round((input_tokens + output_tokens) / elapsed, 1),
        "ttft_ms": snapshot["latency_ms"]["ttft"], "itl_ms": snapshot["latency_ms"]["itl"],
        "e2e_ms": snapshot["latency_ms"]["e2e"], "preempted": snapshot["requests"]["preempted_total"],
        "recomputed_tokens": snapshot["tokens"]["recomputed_total"], "scheduler": snapshot["scheduler"],
        "kv_cache": snapshot.get("kv_cache"), "runner": snapshot.get("runner"), "verified": verified,
        "data": "synthetic (seeded uniform-random token ids, random weights)",
    }


def main(argv: list[str] | None = None) -> int:
    import argparse

    parser = argparse.ArgumentParser(prog="cie workload", description=__doc__.split("\n\n")[0])
    parser.add_argument("name", choices=sorted(PROFILES))
    parser.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has")
    parser.add_argument("--shape", choices=sorted(SHAPES), default=None, help="another model shape than the profile's")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--requests", type=int, default=None, help="another number of requests than the profile's")
    parser.add_argument("--prefill-chunk", type=int, default=None, help="another portion size than the profile's")
    parser.add_argument("--token-budget", type=int, default=None, help="another token budget than the profile's")
    parser.add_argument("--verify", type=int, default=0, metavar="N",
                        help="afterwards run the first N requests alone and compare their tokens "
                             "(float32: must be equal; bfloat16: reported)")
    args = parser.parse_args(argv)
    profile = PROFILES[args.name]
    if args.requests is not None:
        if args.requests < 1:
            parser.error("--requests must be positive")
        profile = replace(profile, requests=args.requests, lead_requests=min(profile.lead_requests, args.requests))
    for option in ("prefill_chunk", "token_budget"):
        value = getattr(args, option)
        if value is not None:
            if value < 1:
                parser.error(f"--{option.replace('_', '-')} must be positive")
            profile = replace(profile, **{option: value})
    record = run_profile(profile, layers=args.layers, dtype=args.dtype, seed=args.seed, shape=args.shape,
                         verify=args.verify)
    print(json.dumps(record))
    return 0
