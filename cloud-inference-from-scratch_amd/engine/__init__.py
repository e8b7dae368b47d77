from .batch import PagedView, StateView, StepBatch
from .engine import Engine, GenerationResult
from .loading import build_model, load_model, random_model
from .runner import Runner, StepEntry
from .scheduler import (
    BatchItem,
    BatchPlan,
    GenerationConfig,
    PreemptionCandidate,
    RejectedError,
    RejectionReason,
    Request,
    RequestState,
    Scheduler,
    SchedulingCandidate,
    decode_first_priority,
    largest_sequence_preemption,
)

__all__ = [
    "BatchItem", "BatchPlan", "Engine", "GenerationConfig", "GenerationResult", "PagedView",
    "PreemptionCandidate", "RejectedError", "RejectionReason", "Request", "RequestState", "Runner",
    "Scheduler", "SchedulingCandidate", "StateView", "StepBatch", "StepEntry", "build_model",
    "decode_first_priority", "largest_sequence_preemption", "load_model", "random_model",
]
