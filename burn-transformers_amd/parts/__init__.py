from . import attention, block, feed_forward, norm, position, readout  # noqa: F401  (registers the parts)
from .base import (Block, Delta, Embedding, FeedForward, Memory, Mixer, Norm, Part, Readout,
                   ResidualStream)
from .registry import lookup, register, unregister

__all__ = ["Block", "Delta", "Embedding", "FeedForward", "Memory", "Mixer", "Norm", "Part",
           "Readout", "ResidualStream", "lookup", "register", "unregister"]
