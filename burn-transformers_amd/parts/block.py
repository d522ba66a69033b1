"""Arrangements of parts in a layer.

pre_norm: y = x + mixer(norm(x)); z = y + feed_forward(norm(y))
(src/models/gpt2/model.rs:218-270).  A part adds its contribution to the stream itself or
returns it as a Delta, which stays pending until the next norm reads the stream.
"""

from .base import Block, offers_chunked
from .registry import register

# Most rows of a step whose first norm is folded too.  Measured at GPT-2 XL sizes, ms a decode step
# without / with it: 1.87 / 1.81 at one row, 1.89 / 1.84 at two, 1.96 / 1.94 at four, 2.14 / 2.23 at
# eight (there the feed-forward's second product misses its split of K more than the norm costs).
# With the limit at eight rows instead, ms a step of eight rows at widths 768 / 1,024 / 1,600 (12, 24
# and 12 layers): 0.395 -> 0.388, 0.781 -> 0.785, 0.531 -> 0.546; so four at every width.
MIXER_FOLD_ROWS = 4


@register("block", "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ff_norm": "norm", "ff": "feed_forward"}
    only_launches_kernels = True

    def forward(self, stream, step, memory):
        parts = self.parts
        mixer, ff, mixer_norm, ff_norm = parts["mixer"], parts["ff"], parts["mixer_norm"], parts["ff_norm"]
        rows = stream.x.shape[0]
        # In a small decode step a norm can be folded into the product that follows it (one kernel
        # fewer) if the part before it leaves its output in the stream itself instead of pending
        # partial sums.  For the second norm that costs the attention output its split of K, which is
        # cheap; for the first norm it costs the feed-forward's second product its split, which pays
        # only for the very smallest steps (MIXER_FOLD_ROWS).
        fold_ff = ff.takes_deferred_norm and _can_defer(ff_norm, step, rows)
        fold_mixer = mixer.takes_deferred_norm and rows <= MIXER_FOLD_ROWS and _can_defer(mixer_norm, step, rows)
        h = mixer_norm.deferred(stream, step) if fold_mixer else None
        if h is None:
            h = _apply(mixer_norm, stream, step, mixer.takes_deferred_norm)
        stream.in_place = fold_ff
        delta = mixer.forward(h, step, memory, stream)
        stream.in_place = False
        if delta is not None:
            stream.add(delta)
        h = ff_norm.deferred(stream, step) if fold_ff else None
        if h is None:
            h = _apply(ff_norm, stream, step, ff.takes_deferred_norm)
        stream.in_place = fold_mixer          # for the next layer's first norm (or the final one, which does not mind)
        delta = ff.forward(h, step, stream)
        stream.in_place = False
        if delta is not None:
            stream.add(delta)


def _apply(norm, stream, step, only_multiplied):
    """The normalised rows; for a part that only hands them to ``gemm``, in the chunk-major layout
    if the norm offers it (the norm decides by the number of rows)."""
    if only_multiplied and offers_chunked(norm):
        return norm.apply(stream, step, chunked=True)
    return norm.apply(stream, step)


def _can_defer(norm, step, rows):
    possible = getattr(norm, "deferred_possible", None)
    return possible is not None and possible(step, rows)
