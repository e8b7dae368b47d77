"""What one scheduler iteration hands to the step function, and the two orders
that a caller may replace.

A plan holds each live request at most once, with the next tokens that request
has not in the cache yet: a portion of a prompt, or the single token it sampled
last (the reference's ``BatchItem``/``BatchPlan``,
src/cloud_engine/scheduler.py:135-166).  The planner's two decisions, which
request runs first and which one gives way when pages run out, are functions of
a read-only :class:`Standing` (the reference shows them as
``scheduling_priority`` and ``preemption_priority`` over two candidate records,
src/cloud_engine/scheduler.py:168-199).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from .request import Request, RequestState


@dataclass(frozen=True)
class Portion:
    """The tokens of one request in one step: ``tokens`` go to positions
    ``start .. start+len-1``; ``samples`` says that they reach the request's
    last known token, so the step's logits there yield its next token."""

    request: Request
    start: int
    tokens: tuple[int, ...]
    samples: bool

    @property
    def length(self) -> int:
        return len(self.tokens)

    @property
    def end(self) -> int:
        return self.start + len(self.tokens)

    @property
    def is_decode(self) -> bool:
        """One token behind the prompt: the token the request sampled last."""
        return len(self.tokens) == 1 and self.start >= len(self.request.prompt)


@dataclass(frozen=True)
class StepPlan:
    portions: tuple[Portion, ...]

    def __bool__(self) -> bool:
        return bool(self.portions)

    @property
    def token_count(self) -> int:
        return sum(portion.length for portion in self.portions)

    @property
    def request_ids(self) -> tuple[str, ...]:
        return tuple(portion.request.request_id for portion in self.portions)

    @property
    def all_decode(self) -> bool:
        return all(portion.is_decode and portion.samples for portion in self.portions)


@dataclass(frozen=True)
class Standing:
    """A request as the two orders see it."""

    request_id: str
    decoding: bool          # its next step is one sampled token
    pending_tokens: int     # known tokens not in the cache
    prompt_tokens: int
    output_tokens: int
    cached_tokens: int
    resident_tokens: int    # tokens the pool holds pages for
    preemptions: int
    arrived_ns: int

    @classmethod
    def of(cls, request: Request, resident_tokens: int = 0) -> "Standing":
        return cls(
            request_id=request.request_id,
            decoding=request.state is RequestState.DECODING and request.pending == 1,
            pending_tokens=request.pending,
            prompt_tokens=len(request.prompt),
            output_tokens=len(request.output),
            cached_tokens=request.cached,
            resident_tokens=resident_tokens,
            preemptions=request.preemptions,
            arrived_ns=request.arrived_ns,
        )


def decodes_before_prompts(standing: Standing) -> tuple[Any, ...]:
    """Sort key of the planner (smallest first; the sort is stable, so requests
    keep their order of admission inside each class)."""
    return (0 if standing.decoding else 1,)


def most_resident_gives_way(standing: Standing) -> tuple[Any, ...]:
    """Key of the request that is preempted when pages run out (largest wins):
    the one that holds most, then the one furthest along, then the latest."""
    return (standing.resident_tokens, standing.cached_tokens, standing.arrived_ns)
