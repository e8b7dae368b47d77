"""The Python entry point: ``Engine(...).generate(prompts, GenerationConfig(...))``.

Counterpart of the reference's ``InferenceEngine`` + ``RequestHandle``
(src/cloud_engine/engine.py:491-802): it owns model, cache, step function and
scheduler and returns ``GenerationResult`` with the reference's fields
(src/cloud_engine/engine.py:48-57).  It is synchronous and takes token ids
first; text needs a ``tokenizer.json`` in the model folder.
"""

from __future__ import annotations

import time
from collections.abc import Callable, Sequence
from dataclasses import dataclass
from pathlib import Path
from typing import Any

from ..config.engine_config import EngineConfig, build_engine_config
from ..metrics import Metrics
from .loading import load_model, random_model
from .runner import Runner
from .plan import decodes_before_prompts, most_resident_gives_way
from .request import GenerationConfig, Request, RequestState
from .scheduler import Scheduler


@dataclass
class GenerationResult:
    request_id: str
    text: str
    token_ids: list[int]
    input_tokens: int
    output_tokens: int
    finish_reason: str
    ttft_ms: float | None
    e2e_ms: float


class Engine:
    """``Engine(model_dir, dtype="bfloat16", ...)`` loads a folder;
    ``Engine(config=typed_config, seed=0, ...)`` makes random weights.  Other
    keyword arguments are :class:`~cie_amd.config.EngineConfig` fields."""

    def __init__(self, model_dir: str | Path | None = None, *, config: Any = None, seed: int = 0,
                 engine_config: EngineConfig | None = None, device: str = "cuda:0",
                 draw_device: str = "cpu",
                 runner_factory: Callable[[EngineConfig], Any] | None = None,
                 plan_order=decodes_before_prompts, victim_order=most_resident_gives_way,
                 **options: Any) -> None:
        self.engine_config = build_engine_config(engine_config, **options)
        self.model_dir = Path(model_dir) if model_dir is not None else None
        self.tokenizer = None
        if runner_factory is not None:
            self.model = None
            self.model_config = config
            self.runner = runner_factory(self.engine_config)
        else:
            if model_dir is not None:
                self.model, self.model_config = load_model(model_dir, self.engine_config.dtype, device)
            elif config is not None:
                self.model = random_model(config, seed, self.engine_config.dtype, device, draw_device)
                self.model_config = config
            else:
                raise ValueError("give a model folder or a configuration for random weights")
            # a request can never be longer than the model's position table
            positions = self.model.spec.max_position
            if self.engine_config.max_model_len > positions:
                self.engine_config = build_engine_config(self.engine_config, max_model_len=positions)
            self.runner = Runner(self.model, self.engine_config, device)
        self.metrics = Metrics()
        self.scheduler = Scheduler(self.engine_config, self.runner, self.metrics,
                                   plan_order=plan_order, victim_order=victim_order)

    # -- text ------------------------------------------------------------------------
    def _tokenizer(self) -> Any:
        if self.tokenizer is None:
            path = self.model_dir / "tokenizer.json" if self.model_dir is not None else None
            if path is None or not path.is_file():
                raise ValueError("text prompts need a tokenizer.json in the model folder; pass token ids instead")
            from tokenizers import Tokenizer

            self.tokenizer = Tokenizer.from_file(str(path))
        return self.tokenizer

    def tokenize(self, prompt: str) -> list[int]:
        return list(self._tokenizer().encode(prompt).ids)

    def detokenize(self, token_ids: Sequence[int]) -> str:
        if self.tokenizer is None and (self.model_dir is None or not (self.model_dir / "tokenizer.json").is_file()):
            return ""
        return self._tokenizer().decode(list(token_ids))

    # -- requests ----------------------------------------------------------------------
    def _generation_config(self, gen: GenerationConfig | None) -> GenerationConfig:
        if gen is not None:
            return gen
        eos = self.engine_config.eos_token_id
        if eos is None and self.model_config is not None:
            eos = getattr(self.model_config, "eos_token_id", None)
        return GenerationConfig(max_output_tokens=self.engine_config.max_output_tokens, eos_token_id=eos)

    def submit(self, prompt: str | Sequence[int], gen: GenerationConfig | None = None,
               on_token: Callable[[Request, int], None] | None = None) -> Request:
        token_ids = self.tokenize(prompt) if isinstance(prompt, str) else list(prompt)
        label = prompt if isinstance(prompt, str) else ""
        return self.scheduler.submit(token_ids, self._generation_config(gen), label=label, on_token=on_token)

    def step(self) -> bool:
        return self.scheduler.step()

    def warm_up(self) -> int:
        """Capture the decode graphs of all bucket sizes before the first request (a serving process
        does this at start; otherwise each bucket is captured by the first step that needs it)."""
        warm = getattr(self.runner, "warm_up", None)
        return warm() if warm is not None else 0

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def result_of(self, request: Request) -> GenerationResult:
        if request.state is not RequestState.COMPLETED:
            raise RuntimeError(f"generation {request.state.value}: {request.error or request.finish_reason}")
        end = request.ended_ns or time.monotonic_ns()
        return GenerationResult(
            request_id=request.request_id,
            text=self.detokenize(request.output),
            token_ids=list(request.output),
            input_tokens=len(request.prompt),
            output_tokens=len(request.output),
            finish_reason=request.finish_reason,
            ttft_ms=(request.first_token_ns - request.arrived_ns) / 1e6 if request.first_token_ns else None,
            e2e_ms=(end - request.arrived_ns) / 1e6,
        )

    def generate(self, prompts: Sequence[str | Sequence[int]],
                 gen: GenerationConfig | Sequence[GenerationConfig] | None = None,
                 on_token: Callable[[Request, int], None] | None = None) -> list[GenerationResult]:
        """Run all prompts to completion, batched by the scheduler; results in the prompts' order."""
        configs = list(gen) if isinstance(gen, (list, tuple)) else [gen] * len(prompts)
        if len(configs) != len(prompts):
            raise ValueError("one GenerationConfig per prompt, or one for all")
        pending = list(zip(prompts, configs))
        requests: list[Request] = []
        while pending or self.scheduler.has_work():
            while pending and len(self.scheduler.waiting) < self.engine_config.max_queue_size:
                prompt, config = pending.pop(0)
                requests.append(self.submit(prompt, config, on_token=on_token))
            self.scheduler.step()
        return [self.result_of(request) for request in requests]

    def snapshot_metrics(self) -> dict[str, Any]:
        snapshot = self.metrics.snapshot()
        runner = self.runner
        cache = getattr(runner, "cache", None)
        if cache is not None:
            stats = cache.stats()
            snapshot["kv_cache"] = {
                "pages_total": stats.pages_total, "pages_used": stats.pages_used,
                "utilization": round(stats.utilization, 4),
                "request_pages_used": stats.request_pages_used, "prefix_pages_used": stats.prefix_pages_used,
                "prefix_cache_hits": stats.prefix_cache_hits, "prefix_cache_misses": stats.prefix_cache_misses,
                "reserved_bytes": stats.reserved_bytes, "occupied_bytes": stats.occupied_bytes,
                "internal_fragmentation_bytes": stats.internal_fragmentation_bytes,
                "groups": [
                    {"units": g.units, "pages_total": g.pages_total, "pages_used": g.pages_used,
                     "reserved_bytes": g.reserved_bytes, "occupied_bytes": g.occupied_bytes,
                     "internal_fragmentation_bytes": g.internal_fragmentation_bytes}
                    for g in stats.groups
                ],
            }
        snapshot["runner"] = {
            "forward_invocations": getattr(runner, "forward_invocations", 0),
            "max_forward_request_count": getattr(runner, "max_forward_request_count", 0),
            "graph_captures": getattr(runner, "graph_captures", 0),
            "graph_replays": getattr(runner, "graph_replays", 0),
            "mixed_graph_captures": getattr(runner, "mixed_graph_captures", 0),
            "mixed_graph_replays": getattr(runner, "mixed_graph_replays", 0),
        }
        return snapshot
