"""A request's record from submission to its end, and what a caller may ask of it.

The life of a request follows the reference's state machine
(src/cloud_engine/scheduler.py:1-13): it waits, its prompt runs in portions, it
decodes token by token, and it ends completed, cancelled or failed.  The token
ids a request has produced are authoritative: after a preemption the cache is
rebuilt from ``prompt + output`` and nothing is sampled twice
(docs/06-ragged-engine.md:47-49 of the reference).
"""

from __future__ import annotations

from collections.abc import Callable
from dataclasses import dataclass, field
from enum import Enum


class RequestState(Enum):
    WAITING = "waiting"
    PREFILL = "prefill"
    DECODING = "decoding"
    COMPLETED = "completed"
    CANCELLED = "cancelled"
    FAILED = "failed"

    @property
    def is_final(self) -> bool:
        return self in (RequestState.COMPLETED, RequestState.CANCELLED, RequestState.FAILED)


class Refusal(Enum):
    """Why a request was not taken at submission (the reference's three reasons,
    src/cloud_engine/scheduler.py:50-53)."""

    QUEUE_FULL = "queue_full"
    NO_CAPACITY = "capacity_exhausted"
    TOO_LONG = "context_length_exceeded"


class RejectedError(RuntimeError):
    def __init__(self, reason: Refusal, detail: str = "") -> None:
        self.reason = reason
        super().__init__(detail if detail else reason.value)


@dataclass
class GenerationConfig:
    """How one request samples and when it stops.

    ``temperature == 0`` takes the largest logit, which is all the reference
    offers (src/cloud_engine/scheduler.py:63-71); a positive temperature draws
    from softmax(logits / temperature) with a random number that depends on
    ``seed`` and the token's index only, never on the batch.  Without an
    ``eos_token_id`` only ``max_output_tokens`` ends the request."""

    max_output_tokens: int
    temperature: float = 0.0
    eos_token_id: int | None = None
    seed: int | None = None

    def __post_init__(self) -> None:
        if self.max_output_tokens < 1:
            raise ValueError("max_output_tokens must be positive")
        if not self.temperature >= 0:
            raise ValueError("temperature must be zero (greedy) or positive")


@dataclass
class Request:
    request_id: str
    serial: int
    prompt: tuple[int, ...]
    gen: GenerationConfig
    arrived_ns: int
    label: str = ""
    on_token: Callable[["Request", int], None] | None = None
    state: RequestState = RequestState.WAITING
    output: list[int] = field(default_factory=list)
    cached: int = 0             # tokens of prompt + output that the cache holds (the runner moves it)
    first_token_ns: int | None = None
    latest_token_ns: int | None = None
    ended_ns: int | None = None
    finish_reason: str = ""
    error: str = ""
    rejected: bool = False
    preemptions: int = 0
    recomputed: int = 0         # tokens run a second time after preemptions
    redo_below: int = 0         # positions under this mark were in the cache before the last preemption

    @property
    def is_final(self) -> bool:
        return self.state.is_final

    @property
    def known(self) -> int:
        """Tokens whose ids are fixed: the prompt and what has been sampled."""
        return len(self.prompt) + len(self.output)

    @property
    def pending(self) -> int:
        """Known tokens that the cache does not hold yet."""
        return self.known - self.cached

    def tokens(self, start: int, end: int) -> tuple[int, ...]:
        """Token ids at positions ``start..end-1`` of prompt + output, without joining the two
        (a decode step would otherwise copy its whole context)."""
        split = len(self.prompt)
        if start >= split:
            return tuple(self.output[start - split: end - split])
        if end <= split:
            return self.prompt[start:end]
        return self.prompt[start:] + tuple(self.output[: end - split])
