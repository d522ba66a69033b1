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
        mixer, ff, ff_norm = parts["mixer"], parts["ff"], parts["ff_norm"]
        # In a small decode step the second norm can be folded into the feed-forward's first product
        # (one kernel fewer a layer) if the mixer leaves its output in the stream itself.
        fold = ff.takes_deferred_norm and getattr(ff_norm, "deferred_possible", None) is not None and \
            ff_norm.deferred_possible(step, stream.x.shape[0])
        stream.in_place = fold
        delta = mixer.forward(parts["mixer_norm"].apply(stream, step), step, memory, stream)
        stream.in_place = False
        if delta is not None:
            stream.add(delta)
        h = ff_norm.deferred(stream, step) if fold else None
        if h is None:
            h = ff_norm.apply(stream, step)
        delta = ff.forward(h, step, stream)
        if delta is not None:
            stream.add(delta)
