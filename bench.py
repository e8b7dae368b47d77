#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens per second of a Qwen2.5 shape
(default: the 3B one) with random weights, plus prefill and roofline figures.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096]
                    [--shape 0.5b|3b|7b|14b|32b|72b] [--layers N] [--long-contexts 32768]
                    [--mixed-portions 16,64,248] [--other-shapes 7b,14b]

A "step" is one decode step of the whole engine (scheduler iteration: plan,
step function, sampling, token hand-over).  Protocol after the reference's
benchmark (benchmarks/run.py:3-8, 205-207, 241-256): a fresh engine per
measured point, two unmeasured warm-up runs, three measured runs, every run
reported and the median taken; wall-clock output tokens per second; prompts are
seeded uniform-random token ids, EOS is ignored.

A *run* of the headline figure is a window of exactly K decode steps between two
``torch.cuda.synchronize()``; the windows follow one another in the same batch
of requests, after W untimed steps, and the last one ends at ``--context``
tokens, so all of them sit at the heavy end of the range that the configuration
states ("2,048-token prefill, then decode to 4,096").  The whole range is
measured beside it (``range``): prompts of ``--prefill-tokens``, then every
decode step up to ``--context``, one warm-up run and three measured ones.
``prefill`` is one prompt of ``--prefill-tokens`` run to its first token.
``mixed`` is the time of the steps that chunked serving meets: the batch's decode
tokens beside one portion of a further prompt (``--mixed-portions``).  ``points``
holds decode at batch 1 and 64, at the main batch behind ``--long-contexts``
tokens, and, for the ``--other-shapes`` of the family, decode at the main batch
and context and the prefill, each with its share of the roofline in
``points_frac`` (the bytes and flops of its own shape).  ONE JSON line is printed.
"""

from __future__ import annotations

import argparse
import gc
import json
import statistics
import sys
import time

# MI355X published peaks.
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

SLACK = 16  # tokens a request may run past the nominal context (requests start decoding a step or two apart)
WARM_WINDOWS = 2
MEASURED_WINDOWS = 3
PAGE = 16


def linear_params_per_layer(c) -> int:
    q = c.num_attention_heads * c.head_dim
    kv = c.num_key_value_heads * c.head_dim
    return c.hidden_size * (q + 2 * kv) + q * c.hidden_size + 3 * c.hidden_size * c.intermediate_size


def decode_bytes(c, layers: int, batch: int, context: float, elem: int) -> float:
    """Bytes one decode step has to read: every weight once, and the cache of the live requests."""
    weights = layers * (linear_params_per_layer(c) + 2 * c.hidden_size
                        + (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim) * elem
    weights += c.vocab_size * c.hidden_size * elem + c.hidden_size * elem  # the head (tied or not: read once) + final norm
    kv = batch * context * layers * 2 * c.num_key_value_heads * c.head_dim * elem
    return weights + kv


def prefill_flops(c, layers: int, tokens: int) -> float:
    linears = 2.0 * tokens * layers * linear_params_per_layer(c)
    attention = layers * 2 * 2 * (tokens * (tokens + 1) / 2) * c.head_dim * c.num_attention_heads
    head = 2.0 * c.hidden_size * c.vocab_size
    return linears + attention + head


def make_engine(config, dtype, batch, context, prefill_tokens, seed=0):
    from cie_amd import Engine

    per_request = -(-(context + SLACK) // PAGE) * PAGE
    kv_tokens = max(batch * per_request, -(-prefill_tokens // PAGE) * PAGE) + 4 * PAGE
    return Engine(
        config=config, seed=seed, dtype=dtype, page_size=PAGE, kv_tokens=kv_tokens,
        max_running=max(batch, 1), max_queue_size=max(batch, 1) + 1, max_model_len=context + SLACK,
        max_output_tokens=context, token_budget=max(2048, batch), prefill_chunk=2048,
        prefix_cache_pages=0, draw_device="cuda",
        # fill all caches before decoding starts, so that the timed steps are pure decode steps
        plan_order=lambda standing: (standing.decoding,),
    )


def random_prompts(config, count: int, length: int, seed: int) -> list[list[int]]:
    import torch

    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, config.vocab_size, (length,), generator=g).tolist() for _ in range(count)]


def decode_windows(engine, config, batch: int, context: int, steps: int, warmup: int, seed: int):
    """``batch`` requests whose last window ends at ``context``: W untimed steps, then
    ``WARM_WINDOWS`` unmeasured and ``MEASURED_WINDOWS`` measured windows of exactly ``steps`` steps.
    Returns [(seconds, mean context of the window)] of the measured ones."""
    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    windows = WARM_WINDOWS + MEASURED_WINDOWS
    prompt_len = context - warmup - windows * steps
    if prompt_len < 1:
        raise ValueError(f"context {context} too short for {warmup} + {windows} x {steps} steps")
    gen = GenerationConfig(max_output_tokens=warmup + windows * steps + SLACK, eos_token_id=None)
    requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, prompt_len, seed)]
    while any(r.state is not RequestState.DECODING for r in requests):
        engine.step()  # prefill portions; the last one yields each request's first token
    for _ in range(warmup - 1):
        engine.step()
    measured = []
    for window in range(windows):
        torch.cuda.synchronize()
        start = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        if window >= WARM_WINDOWS:
            measured.append((elapsed, sum(r.cached for r in requests) / batch - steps / 2.0))
    for r in requests:
        # (with decode steps started ahead of their tokens, the last step's token is still on its way)
        assert not r.is_final and len(r.output) >= warmup + windows * steps - 1, (r.state, len(r.output))
        engine.scheduler.cancel(r)
    return measured


def decode_range(engine, config, batch: int, first: int, last: int, seed: int, warm_steps: int = 48):
    """Prompts of ``first`` tokens, then every decode step until the requests hold ``last`` tokens:
    one short unmeasured run, ``MEASURED_WINDOWS`` measured ones.  Returns [(seconds, decode steps)]."""
    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    out = []
    for run in range(1 + MEASURED_WINDOWS):
        tokens = min(warm_steps, last - first) if run == 0 else last - first
        gen = GenerationConfig(max_output_tokens=tokens, eos_token_id=None)
        requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, first, seed + run)]
        while any(r.state is not RequestState.DECODING for r in requests):
            engine.step()
        torch.cuda.synchronize()
        start = time.perf_counter()
        while engine.has_work():
            engine.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert all(len(r.output) == tokens for r in requests)
        if run:
            out.append((elapsed, tokens - 1))  # the first token came with the prompt
    return out


def mixed_steps(engine, config, batch: int, context: int, portions: list[int], seed: int, steps: int = 24):
    """``batch`` requests decoding near ``context`` tokens; for each portion size, steps that carry
    their tokens and one portion of a long prompt.  Returns {portion: median seconds per step}."""
    import dataclasses

    import torch

    from cie_amd import GenerationConfig
    from cie_amd.engine import RequestState

    settle = 4
    decoded = (len(portions) + 1) * (steps + 2 * settle + 4) + SLACK
    gen = GenerationConfig(max_output_tokens=decoded, eos_token_id=None)
    requests = [engine.submit(prompt, gen) for prompt in random_prompts(config, batch, context - decoded, seed)]
    while any(r.state is not RequestState.DECODING for r in requests):
        engine.step()
    base = engine.scheduler.config
    out = {}
    for portion in portions:
        # the scheduler cuts the long prompt into portions of this size beside the decode tokens
        engine.scheduler.config = dataclasses.replace(base, token_budget=batch + portion, prefill_chunk=portion)
        prompt = random_prompts(config, 1, portion * (steps + settle + 2), seed + portion)[0]
        long = engine.submit(prompt, GenerationConfig(max_output_tokens=1, eos_token_id=None))
        for _ in range(settle):  # (a shape is captured the second time it comes)
            engine.step()
        seconds = []
        for _ in range(steps):
            torch.cuda.synchronize()
            start = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            seconds.append(time.perf_counter() - start)
        assert not long.is_final and all(r.state is RequestState.DECODING for r in requests)
        out[portion] = statistics.median(seconds)
        while not long.is_final:
            engine.step()
    engine.scheduler.config = base
    for r in requests:
        assert not r.is_final
        engine.scheduler.cancel(r)
    return out


def time_prefill(engine, config, tokens: int, seed: int) -> list[float]:
    """Seconds of each measured run: one prompt from submission to its first token."""
    import torch

    from cie_amd import GenerationConfig

    seconds = []
    prompts = random_prompts(config, WARM_WINDOWS + MEASURED_WINDOWS, tokens, seed)
    for run, prompt in enumerate(prompts):
        request = engine.submit(prompt, GenerationConfig(max_output_tokens=1, eos_token_id=None))
        torch.cuda.synchronize()
        start = time.perf_counter()
        while not request.is_final:
            engine.step()
        torch.cuda.synchronize()
        if run >= WARM_WINDOWS:
            seconds.append(time.perf_counter() - start)
    return seconds


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--shape", default="3b", choices=["0.5b", "3b", "7b", "14b", "32b", "72b"])
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in config)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--no-prefill", action="store_true")
    parser.add_argument("--no-range", action="store_true", help="skip the run over the whole range of contexts")
    parser.add_argument("--long-contexts", default=None,
                        help="further decode points of the main batch, e.g. 16384,32768 (default: 32768; none with --no-points)")
    parser.add_argument("--mixed-portions", default=None,
                        help="also time steps of the batch's decode tokens beside a prompt portion of these sizes "
                             "(default 16,64,248; '' for none, as with --no-points)")
    parser.add_argument("--other-shapes", default="7b,14b",
                        help="further shapes whose decode at the main batch and context and whose prefill go into the points ('' for none)")
    args = parser.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not run (this engine is single-GPU)")
        return 2

    import torch

    from cie_amd.config import Qwen2Config
    from cie_amd.workloads import SHAPES

    shape = SHAPES[args.shape]
    full_layers = shape["num_hidden_layers"]
    layers = args.layers or full_layers
    config = Qwen2Config.from_hf_config(dict(shape, num_hidden_layers=layers))
    elem = 2 if args.dtype == "bf16" else 4
    steps, warmup = args.steps, max(args.warmup, 1)

    def release() -> None:
        # (an engine's memory has to be back before the next engine is built: the large shapes fit once)
        gc.collect()
        torch.cuda.empty_cache()

    def say(text: str) -> None:
        print(f"[bench] {text}", file=sys.stderr, flush=True)

    def point(batch: int, context: int, config=config, layers=layers, label: str = ""):
        """(tokens/s of each measured window, the median window's ms per step and roofline share)."""
        context = min(context, config.max_position_embeddings - SLACK)  # (the last positions are the slack's)
        say(f"decode{label}, batch {batch}, context {context}")
        engine = make_engine(config, args.dtype, batch, context, args.prefill_tokens)
        measured = decode_windows(engine, config, batch, context, steps, warmup, seed=batch)
        del engine
        release()
        rates = [batch * steps / seconds for seconds, _ in measured]
        seconds, mean_context = sorted(measured)[len(measured) // 2]
        achieved = decode_bytes(config, layers, batch, mean_context, elem) / (seconds / steps) / 1e9
        return rates, seconds / steps * 1e3, achieved

    def prefill_point(config=config, layers=layers, label: str = ""):
        """(seconds of each measured run, the step's flops) of one prompt run to its first token."""
        say(f"prefill{label} of {args.prefill_tokens} tokens")
        engine = make_engine(config, args.dtype, 1, args.prefill_tokens + 1, args.prefill_tokens)
        seconds = time_prefill(engine, config, args.prefill_tokens, seed=99)
        del engine
        release()
        return seconds, prefill_flops(config, layers, args.prefill_tokens)

    rates, ms_per_step, achieved = point(args.batch, args.context)
    name = f"Qwen2.5-{args.shape.upper()} shape"
    line = {
        "metric": f"decode tokens/s, {name}, batch {args.batch}, context to {args.context}",
        "value": round(statistics.median(rates), 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic (seeded uniform-random token ids, random weights N(0, 0.02))",
        "config": {
            "model": f"{name} (Qwen2ForCausalLM)", "layers": layers, "layers_full": full_layers,
            "hidden": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate": config.intermediate_size, "vocab": config.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": args.prefill_tokens,
            "page_size": PAGE, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings, "attention_bias": config.attention_bias,
            "parallelism": "single GPU",
        },
        "protocol": f"fresh engine per point, {WARM_WINDOWS} unmeasured and {MEASURED_WINDOWS} measured windows of "
                    f"{steps} steps after {warmup} warm-up steps; value is the median window",
        "runs": [round(r, 2) for r in rates],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    if not args.no_range and args.context > args.prefill_tokens + 1:
        say(f"decode over the range {args.prefill_tokens} to {args.context}")
        engine = make_engine(config, args.dtype, args.batch, args.context, args.prefill_tokens)
        runs = decode_range(engine, config, args.batch, args.prefill_tokens, args.context, seed=7)
        del engine
        release()
        range_rates = [args.batch * n / seconds for seconds, n in runs]
        seconds, n = sorted(runs)[len(runs) // 2]
        mean_context = (args.prefill_tokens + args.context) / 2.0
        through = decode_bytes(config, layers, args.batch, mean_context, elem) / (seconds / n) / 1e9
        line["range"] = {
            "from": args.prefill_tokens, "to": args.context, "steps": n,
            "value": round(statistics.median(range_rates), 2), "runs": [round(r, 2) for r in range_rates],
            "ms_per_step": round(seconds / n * 1e3, 4), "frac": round(through / HBM_GBPS, 4),
        }
    if not args.no_prefill:
        seconds, flops = prefill_point()
        median = statistics.median(seconds)
        line["prefill"] = {
            "value": round(args.prefill_tokens / median, 1), "tokens": args.prefill_tokens,
            "ms": round(median * 1e3, 3), "frac": round(flops / median / PEAK_FLOPS[args.dtype], 4),
            "runs_ms": [round(s * 1e3, 3) for s in seconds],
        }
    points, fractions, all_runs = {}, {}, {}
    if not args.no_points:
        for batch in (1, 64):
            rates, _, achieved = point(batch, args.context)
            points[f"decode_b{batch}"] = round(statistics.median(rates), 2)
            fractions[f"decode_b{batch}"] = round(achieved / HBM_GBPS, 4)
            all_runs[f"decode_b{batch}"] = [round(r, 2) for r in rates]
    long_contexts = args.long_contexts if args.long_contexts is not None else ("" if args.no_points else "32768")
    for context in [int(c) for c in long_contexts.split(",") if c]:
        rates, _, achieved = point(args.batch, context)
        key = f"decode_b{args.batch}_ctx{context}"
        points[key] = round(statistics.median(rates), 2)
        fractions[key] = round(achieved / HBM_GBPS, 4)
        all_runs[key] = [round(r, 2) for r in rates]
    # other shapes of the family, whole, at the main batch and context: their own bytes and flops
    if not args.no_points and args.layers is None:
        for other in [name for name in args.other_shapes.split(",") if name and name != args.shape]:
            other_shape = SHAPES[other]
            other_layers = other_shape["num_hidden_layers"]
            other_config = Qwen2Config.from_hf_config(dict(other_shape))
            rates, _, achieved = point(args.batch, args.context, other_config, other_layers, f" ({other} shape)")
            key = f"decode_b{args.batch}_{other}"
            points[key] = round(statistics.median(rates), 2)
            fractions[key] = round(achieved / HBM_GBPS, 4)
            all_runs[key] = [round(r, 2) for r in rates]
            if not args.no_prefill:
                seconds, flops = prefill_point(other_config, other_layers, f" ({other} shape)")
                median = statistics.median(seconds)
                key = f"prefill_{args.prefill_tokens}_{other}"
                points[key] = round(args.prefill_tokens / median, 1)
                fractions[key] = round(flops / median / PEAK_FLOPS[args.dtype], 4)
                all_runs[key] = [round(args.prefill_tokens / s, 1) for s in seconds]
    mixed_portions = args.mixed_portions if args.mixed_portions is not None else ("" if args.no_points else "16,64,248")
    portions = [int(c) for c in mixed_portions.split(",") if c]
    if portions:
        say(f"steps of {args.batch} decode tokens beside a prompt portion of {portions}")
        longest = max(portions)
        engine = make_engine(config, args.dtype, args.batch + 1, max(args.context, 64 * longest), args.prefill_tokens)
        took = mixed_steps(engine, config, args.batch, args.context, portions, seed=5)
        del engine
        release()
        line["mixed"] = {"decoding": args.batch, "context": args.context,
                         "ms_per_step": {str(portion): round(s * 1e3, 4) for portion, s in took.items()}}
    if points:
        line["points"] = points
        line["points_frac"] = fractions
        line["points_runs"] = all_runs
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
