"""Arrangements of parts in a layer.

pre_norm: y = x + mixer(norm(x)); z = y + feed_forward(norm(y))
(src/models/gpt2/model.rs:218-270).  A part adds its contribution to the stream itself or
returns it as a Delta, which stays pending until the next norm reads the stream.
"""

from .base import Block
from .registry import register


@register("block", "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ff_norm": "norm", "ff": "feed_forward"}

    def forward(self, stream, step, memory):
        parts = self.parts
        mixer, ff = parts["mixer"], parts["ff"]
        delta = mixer.forward(parts["mixer_norm"].apply(stream, step), step, memory, stream)
        if delta is not None:
            stream.add(delta)
        delta = ff.forward(parts["ff_norm"].apply(stream, step), step, stream)
        if delta is not None:
            stream.add(delta)
