"""Engine options: the knobs of the reference's ``EngineConfig``
(src/cloud_engine/config.py:24-48, engine_config.json:26-40) that concern one
GPU's engine, under names that say what they bound.  Unknown overrides raise,
as in ``build_config`` (src/cloud_engine/config.py:107-109).
"""

from __future__ import annotations

from dataclasses import dataclass, fields, replace
from typing import Any

DTYPES = ("bfloat16", "float32")
_DTYPE_ALIASES = {"bf16": "bfloat16", "fp32": "float32", "bfloat16": "bfloat16", "float32": "float32"}


def canonical_dtype(name: str) -> str:
    try:
        return _DTYPE_ALIASES[str(name).replace("torch.", "")]
    except KeyError:
        raise ValueError(f"dtype must be one of {DTYPES} (or bf16/fp32), got {name!r}") from None


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"
    max_model_len: int = 4096
    max_output_tokens: int = 256
    eos_token_id: int | None = None
    max_running: int = 16  # reference: max_active_sequences
    max_queue_size: int = 64
    token_budget: int = 2048  # reference: max_batched_tokens
    # the most of one prompt in a step (reference: prefill_chunk_size, 256 there).  On this GPU a step of 264 rows of
    # the 3B shape takes 6.2 ms and one of 2,048 rows 15.5 ms: a prompt cut into eight portions reaches its first
    # token three times later and holds the decoding requests up for longer in sum, so a portion is as long as a step
    prefill_chunk: int = 2048
    page_size: int = 16  # reference: block_size, fixed at 16 there
    kv_tokens: int | None = None  # pool size in tokens; None: from kv_cache_bytes
    # the pool in bytes (the reference's knob, 4 GiB there); None: kv_cache_fraction of the device memory that is
    # free once the weights are loaded.  Either way the pool is no larger than what max_running requests of
    # max_model_len tokens and the prefix index can use.
    kv_cache_bytes: int | None = None
    kv_cache_fraction: float = 0.9
    prefix_cache_pages: int = 256  # reference: prefix_cache_max_blocks
    graph_decode: bool = True  # reference: cuda_graph_decode
    # steps of up to 128 rows that bring prompt portions are captured too, from the second time a shape comes
    # (bucket of the decode rows, lengths of the portions); this many shapes are kept, the least recently used
    # are dropped; 0: such steps always run launch by launch
    graph_mixed_steps: int = 16
    # a captured decode step is started before the tokens of the step before it have reached the host (it takes
    # them on the device); a request that ends on an end-of-sequence token then has run one step too many
    async_decode: bool = True
    # a waiting request is admitted only while the pool has room for the tokens known of it and of every
    # request admitted before it (the reference admits without a look at the pool, src/cloud_engine/scheduler.py:
    # 438-458, and long prompts then evict each other and are computed twice); False: as the reference
    admit_within_pool: bool = True
    # the matrix products of a step that fills the token budget (and of one request's full portion) time every
    # algorithm the vendor library has for their shapes at their first call, a few seconds each, instead of
    # the handful its heuristic proposes; False: the heuristic's candidates only
    search_library_algorithms: bool = True
    seed: int = 0

    def validated(self) -> "EngineConfig":
        config = replace(self, dtype=canonical_dtype(self.dtype))
        for name in ("max_model_len", "max_output_tokens", "max_running", "max_queue_size",
                     "token_budget", "prefill_chunk", "page_size"):
            if getattr(config, name) < 1:
                raise ValueError(f"{name} must be positive")
        if config.page_size & (config.page_size - 1):
            raise ValueError(f"page_size must be a power of two, got {config.page_size}")
        if config.prefix_cache_pages < 0:
            raise ValueError("prefix_cache_pages must be non-negative")
        if config.graph_mixed_steps < 0:
            raise ValueError("graph_mixed_steps must be non-negative")
        if config.kv_tokens is not None and config.kv_tokens < config.page_size:
            raise ValueError("kv_tokens too small for even one page")
        if config.kv_cache_bytes is not None and config.kv_cache_bytes < 1:
            raise ValueError("kv_cache_bytes must be positive")
        if not 0.0 < config.kv_cache_fraction <= 1.0:
            raise ValueError("kv_cache_fraction must lie in (0, 1]")
        return config


# The reference's names (src/cloud_engine/config.py:25-48) of the options that this engine has under a name of
# its own: both are taken, with the same meaning.
REFERENCE_NAMES = {
    "max_active_sequences": "max_running",
    "max_batched_tokens": "token_budget",
    "prefill_chunk_size": "prefill_chunk",
    "block_size": "page_size",
    "prefix_cache_max_blocks": "prefix_cache_pages",
    "cuda_graph_decode": "graph_decode",
}


def build_engine_config(base: EngineConfig | None = None, **overrides: Any) -> EngineConfig:
    for theirs, ours in REFERENCE_NAMES.items():
        if theirs in overrides:
            if ours in overrides:
                raise ValueError(f"{theirs} and {ours} name the same option: give one")
            overrides[ours] = overrides.pop(theirs)
    known = {item.name for item in fields(EngineConfig)}
    unknown = set(overrides) - known
    if unknown:
        raise ValueError(f"unknown config overrides: {sorted(unknown)}")
    return replace(base or EngineConfig(), **overrides).validated()
