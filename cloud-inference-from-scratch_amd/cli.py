"""``cie``: the command line, local instead of the reference's HTTP client.

The reference's ``cie`` (src/cloud_engine/cli.py:53-66) talks to a server:
``health``, ``models``, ``generate PROMPT [--model] [--max-output-tokens 1..256]
[--no-stream]``, ``metrics``.  Here the commands run the engine in-process, so
``--url`` / ``--api-key`` / ``health`` are gone; ``generate`` keeps its options
and their meanings (``--model`` is a folder, env ``ENGINE_MODEL`` still works,
``--max-output-tokens`` defaults to 64, streaming is the default), ``models``
lists the registered architectures, ``metrics`` prints the counters of a run.
Added: ``init-model`` (random-weights mode), ``replay`` (trace replay) and
``bench``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _engine_options(parser: argparse.ArgumentParser) -> None:
    parser.add_argument("--model", default=os.environ.get("ENGINE_MODEL"),
                        help="model folder (config.json + *.safetensors); env ENGINE_MODEL")
    parser.add_argument("--random-weights", metavar="CONFIG_JSON",
                        help="instead of --model: a config.json to run with seeded random weights")
    parser.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    # (engine options that are not given keep the engine's defaults)
    parser.add_argument("--page-size", type=int, default=None, help="tokens per cache page (a power of two)")
    parser.add_argument("--kv-tokens", type=int, default=None, help="cache pool size in tokens")
    parser.add_argument("--kv-pages", type=int, default=None, help="cache pool size in pages, instead of --kv-tokens")
    parser.add_argument("--token-budget", type=int, default=None, help="most tokens in a step")
    parser.add_argument("--prefill-chunk", type=int, default=None, help="most tokens of one prompt in a step")
    parser.add_argument("--max-running", type=int, default=None, help="most requests that hold cache at a time")
    parser.add_argument("--max-model-len", type=int, default=None)


def parser() -> argparse.ArgumentParser:
    cli = argparse.ArgumentParser(prog="cie", description=__doc__,
                                  formatter_class=argparse.RawDescriptionHelpFormatter)
    commands = cli.add_subparsers(dest="command", required=True)
    commands.add_parser("models", help="list the registered architectures")
    generate = commands.add_parser("generate", help="generate tokens")
    generate.add_argument("prompt", nargs="?", help="text (needs tokenizer.json in the model folder)")
    generate.add_argument("--token-ids", help="comma or space separated prompt token ids")
    generate.add_argument("--max-output-tokens", type=int, default=64)
    generate.add_argument("--temperature", type=float, default=0.0)
    generate.add_argument("--ignore-eos", action="store_true")
    generate.add_argument("--no-stream", action="store_true")
    generate.add_argument("--metrics", action="store_true", help="print the run's metrics as JSON afterwards")
    _engine_options(generate)
    metrics = commands.add_parser("metrics", help="run a prompt and print only the metrics as JSON")
    metrics.add_argument("--token-ids", default="1 2 3 4 5 6 7 8")
    metrics.add_argument("--max-output-tokens", type=int, default=16)
    _engine_options(metrics)
    init = commands.add_parser("init-model", help="write a model folder with random weights")
    init.add_argument("--config", required=True, help="a config.json")
    init.add_argument("--out", required=True)
    init.add_argument("--seed", type=int, default=0)
    init.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    replay = commands.add_parser("replay", help="trace replay (bin/trace_run)", add_help=False)
    replay.add_argument("rest", nargs=argparse.REMAINDER)
    bench = commands.add_parser("bench", help="the serving benchmark (bench.py)", add_help=False)
    bench.add_argument("rest", nargs=argparse.REMAINDER)
    commands.add_parser("ceilings", help="memory bandwidth and bf16 matrix throughput this GPU reaches")
    workload = commands.add_parser("workload", help="an offline serving workload with random weights", add_help=False)
    workload.add_argument("rest", nargs=argparse.REMAINDER)
    return cli


def _make_engine(args: argparse.Namespace):
    from .config import config_from_dict
    from .engine import Engine

    from .config.engine_config import EngineConfig

    if args.kv_pages is not None and args.kv_tokens is not None:
        raise SystemExit("cie: --kv-pages and --kv-tokens both size the cache pool: give one")
    options = dict(dtype=args.dtype, seed=args.seed)
    for name in ("page_size", "kv_tokens", "token_budget", "prefill_chunk", "max_running", "max_model_len"):
        if getattr(args, name) is not None:
            options[name] = getattr(args, name)
    if args.kv_pages is not None:
        options["kv_tokens"] = args.kv_pages * options.get("page_size", EngineConfig.page_size)
    if args.random_weights:
        with open(args.random_weights, encoding="utf-8") as handle:
            config = config_from_dict(json.load(handle))
        options.pop("seed")
        return Engine(config=config, seed=args.seed, **options)
    if not args.model:
        raise SystemExit("cie: --model DIR (or ENGINE_MODEL) or --random-weights CONFIG_JSON is required")
    return Engine(args.model, **options)


def _token_ids(text: str) -> list[int]:
    return [int(piece) for piece in text.replace(",", " ").split()]


def _run_script(path: Path, rest: list[str]) -> int:
    import runpy

    sys.argv = [str(path), *[r for r in rest if r != "--"]]
    try:
        runpy.run_path(str(path), run_name="__main__")
    except SystemExit as exc:
        return int(exc.code or 0)
    return 0


def main(argv: list[str] | None = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] in ("replay", "bench", "workload", "ceilings"):
        # these hand all their options on; argparse would claim the ones that start with a dash
        args = argparse.Namespace(command=argv[0], rest=argv[1:])
    else:
        args = parser().parse_args(argv)
    if args.command == "models":
        from .config import ARCHITECTURES

        print(json.dumps({"architectures": sorted(ARCHITECTURES)}, indent=2))
        return 0
    if args.command == "init-model":
        from .config import config_from_dict
        from .weights import write_model_folder

        with open(args.config, encoding="utf-8") as handle:
            config = config_from_dict(json.load(handle))
        print(write_model_folder(args.out, config, args.seed, args.store_dtype))
        return 0
    if args.command == "replay":
        return _run_script(ROOT / "bin" / "trace_run", args.rest)
    if args.command == "bench":
        return _run_script(ROOT / "bench.py", args.rest)
    if args.command == "ceilings":
        from .ceilings import main as ceilings_main

        return ceilings_main(args.rest)
    if args.command == "workload":
        from .workloads import main as workload_main

        return workload_main([r for r in args.rest if r != "--"])

    from .engine import GenerationConfig

    engine = _make_engine(args)
    if args.command == "metrics":
        engine.generate([_token_ids(args.token_ids)], GenerationConfig(max_output_tokens=args.max_output_tokens))
        print(json.dumps(engine.snapshot_metrics(), indent=2))
        return 0
    if args.token_ids:
        prompt: object = _token_ids(args.token_ids)
    elif args.prompt is not None:
        prompt = args.prompt
    else:
        raise SystemExit("cie generate: give PROMPT or --token-ids")
    eos = None if args.ignore_eos else getattr(engine.model_config, "eos_token_id", None)
    gen = GenerationConfig(max_output_tokens=args.max_output_tokens, temperature=args.temperature,
                           eos_token_id=eos, seed=args.seed if args.temperature > 0 else None)
    as_text = isinstance(prompt, str)
    streaming = not args.no_stream

    def on_token(request, token_id: int) -> None:
        piece = engine.detokenize([token_id]) if as_text else f"{token_id} "
        print(piece, end="", flush=True)

    result = engine.generate([prompt], gen, on_token=on_token if streaming else None)[0]
    if streaming:
        print()
    else:
        print(result.text if as_text else " ".join(map(str, result.token_ids)))
    if args.metrics:
        print(json.dumps(engine.snapshot_metrics(), indent=2))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
