"""The interfaces the parts of a layer meet, and the residual stream they work on.

  Norm         apply(stream, step, rows=None) -> normalised activations [tokens, width]
  Mixer        forward(h, step, memory) -> Delta         (attention here; anything that mixes tokens)
               kv_spec() / state_spec() say what it keeps in the cache, per token / per sequence
  FeedForward  forward(h, step) -> Delta
  Embedding    embed(step) -> ResidualStream             (token table and position encoding)
  Readout      logits(h, step) -> float32 [rows, vocab]
  Block        forward(stream, step, memory)             (the arrangement of the parts above)

No part knows which model it is in: it gets its sizes and constants as parameters and its
tensors by role from the weight store.

The residual stream is kept in float32 in both precisions.  A part adds to it in one of two
ways: ``stream.add_product(step, a, weight, bias)`` lets the matrix product's epilogue add into
the stream directly (or, where splitting K pays, leaves 32-bit partial sums pending), and
``stream.add(Delta)`` leaves any float32 tensor pending; what is pending is added by the next
norm while it reads the stream anyway.
"""

import functools
from dataclasses import dataclass
from typing import Optional

import torch

from ..kernels import library as K


@dataclass
class Delta:
    """A contribution to the residual stream that has not been added yet:
    sum(partials, dim 0) + bias.  partials: float32 [splits, tokens, width]."""
    partials: torch.Tensor
    bias: Optional[torch.Tensor] = None


class ResidualStream:
    def __init__(self, x):
        self.x = x              # float32 [tokens, width]
        self.pending = None     # Delta or None
        # set by a block around a part whose output the next norm wants in the stream itself, not
        # pending beside it (the norm is then folded into the product that follows it)
        self.in_place = False

    def add(self, delta):
        if self.pending is not None:
            self.flush()
        self.pending = delta

    def add_product(self, step, a, weight, bias=None, packed=None):
        """x += a . weight^T + bias.  In a decode step (up to 64 rows) a product with few
        output columns splits its K range into partial sums that stay pending: the extra work-groups
        are needed to pull the matrix through HBM; so does a bfloat16 product of a short prompt or
        chunk (``kernels.library.deep_split_count``).  Otherwise the product's epilogue adds into the
        stream in place.  ``packed``: the weight's ``kernels.library.PackedWeight``, if it has one."""
        rows, width = a.shape[0], weight.shape[0]
        if self.in_place:
            splits = 1
        elif step.dtype_is_bf16 and rows > 64:       # a short prompt or chunk: the tile kernel's deep forms
            splits = K.deep_split_count(rows, width, a.shape[1], compute_units(a.device)) \
                if not isinstance(a, K.Chunked) and a.stride(1) == 1 and \
                K.deep_form_rows(rows, a.shape[1], a.stride(0), width, sliced=True) else 1
        elif step.dtype_is_bf16:
            splits = split_count(rows, width, a.shape[1], compute_units(a.device), 32)
        elif a.shape[1] % 4 == 0 and a.stride(0) % 4 == 0:        # what the float32 MFMA kernels take
            splits = split_count(rows, width, a.shape[1], compute_units(a.device), 16)
        else:
            splits = 1
        if splits > 1:
            partials = step.partial_sums("stream.partials", splits, rows, width)
            K.gemm(a, weight, K.epilogue_f32(partials), splits=splits, packed=packed)
            self.add(Delta(partials, bias))
        else:
            self.flush()
            K.gemm(a, weight, K.epilogue_residual(self.x, bias), packed=packed)

    def flush(self):
        """Adds what is pending without normalising anything."""
        if self.pending is not None:
            K.add_norm(self.x, None, None, None, 0.0, delta=self.pending.partials, bias=self.pending.bias)
            self.pending = None


class Memory:
    """What a mixer gets of the cache for one run of its layer."""

    def __init__(self, cache, entry, writes, step):
        self.cache, self.entry, self.writes, self.step = cache, entry, writes, step

    def kv(self):
        """Kernel view of this entry's keys and values with the step's block table."""
        return self.cache.kv_view(self.entry, self.step.block_table)

    def state(self):
        """[slots, *shape] per-sequence state of this entry; rows ``step.slots`` are the step's."""
        return self.cache.state(self.entry)


class Part:
    # True for a part whose step does nothing but call kernels of ``kernels.library`` with
    # arguments that depend only on the step's shape and on addresses that stay where they are
    # (weights, the step's workspaces and tables): the engine then keeps a step's calls as a launch
    # list and walks it in C++ (``kernels.library.Program``).  A part that computes with torch,
    # reads the step's host tables or allocates in its step leaves this False, and every step of a
    # model that holds such a part is issued from Python, call by call.
    only_launches_kernels = False

    def __init__(self, params, tensors):
        self.params, self.tensors = params, tensors

    def kernel_modules(self, dtype):
        """Names of kernel modules (``kernels.build.register_module``) that must be built and loaded
        before this part's first step, beyond those every model uses: what the part's own kernels
        live in.  They are compiled side by side when the model is built."""
        return ()


class Norm(Part):
    def apply(self, stream, step, rows=None):
        """Normalised rows as a tensor [rows, width] in the step's dtype.  A norm may take a fourth
        argument ``chunked``: when the block sets it, the part that follows only hands the rows to
        ``kernels.library.gemm`` (``takes_deferred_norm``), and the norm may return them as a
        ``kernels.library.Chunked``, the layout the product of a small step reads fastest."""
        raise NotImplementedError

    def deferred(self, stream, step):
        """The stream's rows as an operand that the next product normalises itself
        (``kernels.library.Normalized``), or None where this norm, this step or what is pending on
        the stream does not allow it; the caller then calls ``apply``."""
        return None


_chunked_norms = {}


def offers_chunked(norm):
    """Whether a norm's ``apply`` takes the ``chunked`` argument (see :class:`Norm`)."""
    kind = type(norm)
    if kind not in _chunked_norms:
        import inspect
        _chunked_norms[kind] = "chunked" in inspect.signature(kind.apply).parameters
    return _chunked_norms[kind]


class Mixer(Part):
    # True for a mixer that hands ``h`` to ``kernels.library.gemm`` and looks at nothing but its
    # shape (see FeedForward.takes_deferred_norm)
    takes_deferred_norm = False
    # False for a mixer whose forward reads the step's host tables (``step.host``) or otherwise
    # does per-step work in Python: steps of a model with such a mixer are never graph-replayed
    graph_safe = True

    def kv_spec(self):
        return None

    def state_spec(self):
        return None

    def forward(self, h, step, memory, stream):
        """Adds the mixer's contribution to ``stream`` (or returns it as a Delta)."""
        raise NotImplementedError


class FeedForward(Part):
    # True for a feed-forward that hands ``h`` to ``kernels.library.gemm`` and looks at nothing
    # but its shape: it may then get rows that are still to be normalised (Norm.deferred)
    takes_deferred_norm = False

    def forward(self, h, step, stream):
        """Adds the feed-forward's contribution to ``stream`` (or returns it as a Delta)."""
        raise NotImplementedError


class Embedding(Part):
    def embed(self, step):
        raise NotImplementedError


class Readout(Part):
    # True for a readout that hands ``h`` to ``kernels.library.gemm`` and looks at nothing but its shape
    takes_deferred_norm = False

    def logits(self, h, step):
        raise NotImplementedError


class Block:
    """An arrangement of parts.  ``ROLES`` maps the block's own names for its parts to the registry
    each is looked up in ("mixer", "feed_forward", "norm"); the names are the block's business, and
    the engine asks the block, not the names, what it needs."""

    ROLES = {}
    only_launches_kernels = False       # as for a part: True if ``forward`` only calls its parts and the stream

    def __init__(self, parts):
        self.parts = parts

    def recordable(self):
        """Whether a step of this block can be kept as a launch list."""
        return self.only_launches_kernels and all(part.only_launches_kernels for part in self.parts.values())

    def mixers(self):
        """The parts of this block that mix tokens (they say what the cache has to keep and which
        kernels have to be built), whatever the block calls them."""
        return [part for part in self.parts.values() if isinstance(part, Mixer)]

    def cache_needs(self):
        """(KVSpec or None, StateSpec or None): what one run of this block keeps in its cache entry.
        A block has one cache entry per run, so at most one of its mixers may keep keys and values
        and at most one fixed-size state."""
        kv = [spec for spec in (mixer.kv_spec() for mixer in self.mixers()) if spec is not None]
        state = [spec for spec in (mixer.state_spec() for mixer in self.mixers()) if spec is not None]
        if len(kv) > 1 or len(state) > 1:
            raise ValueError(f"{type(self).__name__}: a block's run has one cache entry, but several of its "
                             f"mixers keep keys and values or state; give each of them a layer of its own")
        return (kv[0] if kv else None, state[0] if state else None)

    def forward(self, stream, step, memory):
        raise NotImplementedError


@functools.lru_cache(maxsize=None)
def compute_units(device):
    return torch.cuda.get_device_properties(device).multi_processor_count


def packed_for_stream(weight):
    """A matrix's packed copy for the product that adds to the residual stream in decode steps
    (laid out for the split of K such steps use, and for none)."""
    chunk = 32 if weight.dtype == torch.bfloat16 else 16
    splits = 1
    if weight.dtype == torch.bfloat16 or weight.shape[1] % 4 == 0:
        splits = split_count(K.PackedWeight.ROWS, weight.shape[0], weight.shape[1], compute_units(weight.device), chunk)
    return K.PackedWeight(weight, (splits, 1))       # (without a split where the norm behind it is folded)


# What a slice costs beyond the product itself, in the units of ``split_count`` (a work-group's time
# for one chunk of K): the norm behind the product reads every slice's partial sums.  Measured as ms
# a decode step with 0 / 1 / 2 / 3 (12 layers of width 768, 24 of width 1,024, 12 of width 1,600): 24
# rows 0.512 / 0.506 / 0.501 / 0.498, 1.061 / 1.039 / 1.047 / 1.055 and 0.756 / 0.755 / 0.758 / 0.755; 64
# rows 0.707 / 0.699 / 0.695 / 0.694, 1.598 / 1.566 / 1.585 / 1.598 and 1.198 / 1.196 / 1.199 / 1.197 (at
# width 1,024 a step of 17 rows cut K = 1,024 into eight slices of four chunks without it).
SPLIT_READ_COST = 1


def split_count(rows, columns, k, units=256, chunk=32):
    """How many ways a residual-writing product splits its K range (up to 64 rows; 1 beyond).

    The skinny product gives one work-group 16 output columns (32 beyond 16 rows) and one slice
    of K, and its time is set by the compute unit that has to pull the most bytes: a unit takes a work-group of
    ``per`` chunks (``chunk`` K values: 32 of bfloat16, 16 of float32) in about ``per + 10`` units of time (the ten are the work-group's own
    start and its reduction), and ``tiles * splits`` work-groups land on ``units`` compute units
    in whole rounds.  Measured on 100 tiles: K 6400 takes 13.9 / 8.6 / 8.5 / 7.6 / 9.3 us with
    1 / 2 / 4 / 5 / 8 splits, K 1600 takes 5.0 / 4.1 / 4.2 / 4.1 / 5.2 us; the model picks 5 and 2.
    """
    if rows > 64:
        return 1
    tiles = (columns + 15) // 16 if rows <= 16 else (columns + 31) // 32   # beyond 16 rows: 32 columns each
    chunks = (k + chunk - 1) // chunk
    best, best_cost = 1, None
    for splits in range(1, 9):
        per = (chunks + splits - 1) // splits
        if splits > 1 and (per < 4 or per * (splits - 1) >= chunks):    # slices too thin, or an empty one
            continue
        rounds = (tiles * splits + units - 1) // units
        cost = rounds * (per + 10) + SPLIT_READ_COST * splits
        if best_cost is None or cost < best_cost:
            best, best_cost = splits, cost
    return best
