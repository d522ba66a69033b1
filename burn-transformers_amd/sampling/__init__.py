from .config import GenerationConfig, GenerationError
from .tracker import (FinishReason, GeneratedSequence, GenerationTracker, required_capacity,
                      stop_decision)

__all__ = ["GenerationConfig", "GenerationError", "FinishReason", "GeneratedSequence",
           "GenerationTracker", "required_capacity", "stop_decision", "Sampler"]


def __getattr__(name):
    if name in ("Sampler", "splitmix64", "interior_unit"):
        from . import sampler
        return getattr(sampler, name)
    raise AttributeError(name)
