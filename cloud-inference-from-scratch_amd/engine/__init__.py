from .batch import PagedView, StateView, StepBatch
from .engine import Engine, GenerationResult
from .loading import build_model, load_model, random_model
from .plan import Portion, Standing, StepPlan, decodes_before_prompts, most_resident_gives_way
from .request import GenerationConfig, Refusal, RejectedError, Request, RequestState
from .runner import Runner, StepEntry
from .scheduler import Scheduler

__all__ = [
    "Engine", "GenerationConfig", "GenerationResult", "PagedView", "Portion", "Refusal", "RejectedError",
    "Request", "RequestState", "Runner", "Scheduler", "Standing", "StateView", "StepBatch", "StepEntry",
    "StepPlan", "build_model", "decodes_before_prompts", "load_model", "most_resident_gives_way", "random_model",
]
