#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens per second of the Qwen2.5-3B
shape with random weights, plus prefill and roofline figures.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers 36]

A "step" is one decode step of the whole engine (scheduler iteration: plan,
step function, sampling, token hand-over).  The run fills the cache of ``batch``
requests so that the timed steps end at ``context`` tokens, does W untimed and
exactly K timed steps bracketed by ``torch.cuda.synchronize()``, and prints ONE
JSON line.  Protocol after the reference's benchmark (benchmarks/run.py:3-8,
205-207, 241-256): fresh engine, untimed warm-up, wall-clock output tokens per
second; prompts are seeded uniform-random token ids, EOS is ignored.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

# MI355X published peaks.
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

SLACK = 16  # tokens a request may run past the nominal context (requests start decoding a step or two apart)

SHAPE_3B = dict(
    model_type="qwen2", hidden_size=2048, num_hidden_layers=36, num_attention_heads=16,
    num_key_value_heads=2, intermediate_size=11008, vocab_size=151936, rope_theta=1e6,
    rms_norm_eps=1e-6, attention_bias=True, tie_word_embeddings=True, use_sliding_window=False,
    max_position_embeddings=32768, eos_token_id=151643,
)


def linear_params_per_layer(c) -> int:
    q = c.num_attention_heads * c.head_dim
    kv = c.num_key_value_heads * c.head_dim
    return c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size


def decode_bytes(c, layers: int, batch: int, context: float, elem: int) -> float:
    """Bytes one decode step has to read: every weight once, and the cache of the live requests."""
    weights = layers * (linear_params_per_layer(c) + 2 * c.hidden_size
                        + (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim) * elem
    weights += c.vocab_size * c.hidden_size * elem + c.hidden_size * elem  # head (tied: the embedding) + final norm
    kv = batch * context * layers * 2 * c.num_key_value_heads * c.head_dim * elem
    return weights + kv


def prefill_flops(c, layers: int, tokens: int) -> float:
    linears = 2.0 * tokens * layers * linear_params_per_layer(c)
    attention = layers * 2 * 2 * (tokens * (tokens + 1) / 2) * c.head_dim * c.num_attention_heads
    head = 2.0 * c.hidden_size * c.vocab_size
    return linears + attention + head


def make_engine(config, dtype, batch, context, prefill_tokens, seed=0):
    from cie_amd import Engine

    page = 16
    per_request = -(-(context + SLACK) // page) * page
    kv_tokens = max(batch * per_request, -(-prefill_tokens // page) * page) + 4 * page
    return Engine(
        config=config, seed=seed, dtype=dtype, page_size=page, kv_tokens=kv_tokens,
        max_running=max(batch, 1), max_queue_size=max(batch, 1) + 1, max_model_len=context + SLACK,
        max_output_tokens=context, token_budget=max(2048, batch), prefill_chunk=2048,
        prefix_cache_pages=0, draw_device="cuda",
        # fill all caches before decoding starts, so that the timed steps are pure decode steps
        plan_order=lambda standing: (standing.decoding,),
    )


def time_decode(engine, config, batch: int, context: int, steps: int, warmup: int, seed: int):
    """Fill ``batch`` requests so that warm-up plus timed steps end at ``context``; time the steps."""
    import torch

    from cie_amd import GenerationConfig

    prompt_len = context - steps - warmup
    if prompt_len < 1:
        raise ValueError(f"context {context} too short for {steps}+{warmup} steps")
    g = torch.Generator().manual_seed(seed)
    gen = GenerationConfig(max_output_tokens=steps + warmup + SLACK, eos_token_id=None)
    requests = [
        engine.submit(torch.randint(0, config.vocab_size, (prompt_len,), generator=g).tolist(), gen)
        for _ in range(batch)
    ]
    from cie_amd.engine import RequestState

    while any(r.state is not RequestState.DECODING for r in requests):
        engine.step()  # prefill portions; the last one yields each request's first token
    for _ in range(warmup - 1):
        engine.step()
    torch.cuda.synchronize()
    start = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    for r in requests:
        # (with decode steps started ahead of their tokens, the last step's token is still on its way)
        assert not r.is_final and len(r.output) >= warmup + steps - 1, (r.state, len(r.output))
    mean_context = sum(r.cached for r in requests) / batch - steps / 2.0
    for r in requests:
        engine.scheduler.cancel(r)
    return elapsed, mean_context


def time_prefill(engine, config, tokens: int, seed: int, repeats: int = 3):
    import torch

    from cie_amd import GenerationConfig

    g = torch.Generator().manual_seed(seed)
    best = None
    for _ in range(repeats + 1):  # the first is the warm-up
        prompt = torch.randint(0, config.vocab_size, (tokens,), generator=g).tolist()
        request = engine.submit(prompt, GenerationConfig(max_output_tokens=1, eos_token_id=None))
        torch.cuda.synchronize()
        start = time.perf_counter()
        while not request.is_final:
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        best = elapsed if best is None or _ == 1 else min(best, elapsed)
    return best


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--layers", type=int, default=SHAPE_3B["num_hidden_layers"])
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--no-prefill", action="store_true")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not run (this engine is single-GPU)")
        return 2

    import torch

    from cie_amd.config import Qwen2Config

    raw = dict(SHAPE_3B, num_hidden_layers=args.layers)
    config = Qwen2Config.from_hf_config(raw)
    elem = 2 if args.dtype == "bf16" else 4
    full_layers = SHAPE_3B["num_hidden_layers"]

    def decode_point(batch: int, steps: int, warmup: int):
        engine = make_engine(config, args.dtype, batch, args.context, args.prefill_tokens)
        elapsed, mean_context = time_decode(engine, config, batch, args.context, steps, warmup, seed=batch)
        del engine
        torch.cuda.empty_cache()
        return elapsed, mean_context

    elapsed, mean_context = decode_point(args.batch, args.steps, max(args.warmup, 1))
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    achieved = decode_bytes(config, args.layers, args.batch, mean_context, elem) / (elapsed / args.steps) / 1e9
    line = {
        "metric": f"decode tokens/s, Qwen2.5-3B shape, batch {args.batch}, context to {args.context}",
        "value": round(value, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": max(args.warmup, 1),
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic (seeded uniform-random token ids, random weights N(0, 0.02))",
        "config": {
            "model": "Qwen2.5-3B shape (Qwen2ForCausalLM)", "layers": args.layers, "layers_full": full_layers,
            "hidden": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate": config.intermediate_size, "vocab": config.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": args.prefill_tokens,
            "page_size": 16, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings, "attention_bias": config.attention_bias,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    if not args.no_prefill:
        engine = make_engine(config, args.dtype, 1, args.prefill_tokens + 1, args.prefill_tokens)
        seconds = time_prefill(engine, config, args.prefill_tokens, seed=99)
        del engine
        torch.cuda.empty_cache()
        flops = prefill_flops(config, args.layers, args.prefill_tokens)
        line["prefill"] = {
            "value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
            "ms": round(seconds * 1e3, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
        }
    if not args.no_points:
        points = {}
        for batch in (1, 64):
            steps = max(8, args.steps // 2)
            elapsed, _ = decode_point(batch, steps, 4)
            points[f"decode_b{batch}"] = round(batch * steps / elapsed, 2)
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
