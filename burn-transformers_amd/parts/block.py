"""Arrangements of parts in a layer.

pre_norm: y = x + mixer(norm(x)); z = y + feed_forward(norm(y))
(src/models/gpt2/model.rs:218-270).  Each contribution is left pending on the stream and
added by the norm that reads the stream next.
"""

from .base import Block
from .registry import register


@register("block", "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ff_norm": "norm", "ff": "feed_forward"}

    def forward(self, stream, step, memory):
        parts = self.parts
        stream.add(parts["mixer"].forward(parts["mixer_norm"].apply(stream, step), step, memory))
        stream.add(parts["ff"].forward(parts["ff_norm"].apply(stream, step), step))
