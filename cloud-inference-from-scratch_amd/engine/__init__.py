from .batch import PagedView, StateView, StepBatch
from .loading import build_model, load_model, random_model
from .runner import Runner, StepEntry

__all__ = ["PagedView", "Runner", "StateView", "StepBatch", "StepEntry", "build_model", "load_model", "random_model"]
