"""One step's batch as the parts and kernels see it.

A step is a set of sequences, each bringing ``count`` new tokens that start at position
``start`` (its length so far).  Tokens are packed without padding; every token knows its
sequence and position.  All integer tables of a step travel to the GPU in ONE copy, as
sections of one int32 buffer:

    tok_ids[T] tok_pos[T] tok_seq[T] seq_off[B+1] seq_start[B] slots[B] sel_rows[R] block_table[G*B*max_blocks]

(G: the groups of layers of the cache, each with a block table of its own.)
"""

import numpy as np
import torch

from ..cache.ledger import BLOCK


def _align(n):
    return (n + 3) & ~3


class StepLayout:
    """Offsets of the sections for T tokens, B sequences, R wanted rows."""

    def __init__(self, tokens, seqs, rows, max_blocks, groups=1):
        self.tokens, self.seqs, self.rows, self.max_blocks, self.groups = tokens, seqs, rows, max_blocks, groups
        offset = 0
        self.sections = {}
        for name, size in (("tok_ids", tokens), ("tok_pos", tokens), ("tok_seq", tokens),
                           ("seq_off", seqs + 1), ("seq_start", seqs), ("slots", seqs),
                           ("sel_rows", rows), ("block_table", groups * seqs * max_blocks)):
            self.sections[name] = (offset, size)
            offset = _align(offset + size)
        self.total = offset

    def key(self):
        return (self.tokens, self.seqs, self.rows, self.max_blocks, self.groups)


class StepPlan:
    """A validated step on the host: nothing on the GPU or in the cache has changed yet."""

    def __init__(self, slots, starts, counts, token_ids, wanted, block_rows, max_blocks):
        """``block_rows[group][sequence]``: the blocks of each of the step's sequences in each group
        of the cache (``Cache.block_rows``)."""
        self.slots, self.starts, self.counts = slots, starts, counts
        self.n_seqs, self.n_tokens = len(slots), int(sum(counts))
        self.max_count = int(max(counts))
        self.decode = self.max_count == 1
        groups = max(len(block_rows), 1)
        self.layout = StepLayout(self.n_tokens, self.n_seqs, len(wanted), max_blocks, groups)
        host = np.zeros(self.layout.total, dtype=np.int32)
        section = lambda name: host[self.layout.sections[name][0]:sum(self.layout.sections[name])]
        section("tok_ids")[:] = token_ids
        if self.decode:          # one token each: a token's place in the step is its sequence's
            section("tok_pos")[:] = starts
            section("tok_seq")[:] = np.arange(self.n_seqs, dtype=np.int32)
            section("seq_off")[:] = np.arange(self.n_seqs + 1, dtype=np.int32)
        else:
            section("tok_pos")[:] = np.concatenate([np.arange(s, s + c) for s, c in zip(starts, counts)])
            section("tok_seq")[:] = np.repeat(np.arange(self.n_seqs), counts)
            section("seq_off")[:] = np.concatenate([[0], np.cumsum(counts)])
        section("seq_start")[:] = starts
        section("slots")[:] = slots
        section("sel_rows")[:] = wanted
        table = section("block_table").reshape(groups, self.n_seqs, max_blocks)
        for group, rows in enumerate(block_rows):
            for row, blocks in enumerate(rows):
                table[group, row, :len(blocks)] = blocks
        self.host = host
        self.device_tokens = None      # set by the engine: the tokens, where they are on the GPU already
        self.new_lengths = {slot: start + count for slot, start, count in zip(slots, starts, counts)}
        self.context_limit = min(context_limit(max(self.new_lengths.values())), max_blocks * BLOCK)


SHORT_CONTEXT = 1024


def context_limit(longest):
    """The class of a step by its longest sequence: SHORT_CONTEXT tokens, then powers of two (and never
    more than a sequence can hold).  Parts
    that plan their work by the context (attention cuts long contexts into runs) plan for this
    bound instead of the exact lengths, so that a step's kernels depend only on its class, and a
    captured graph serves every step of the same class."""
    limit = SHORT_CONTEXT
    while limit < longest:
        limit *= 2
    return limit


class Step:
    """The step on the GPU: views into the device copy of the plan's integer tables, plus the
    workspace the parts draw their buffers from."""

    def __init__(self, plan_or_layout, device_meta, pool, dtype, host_plan=None):
        layout = plan_or_layout
        self.n_tokens, self.n_seqs, self.max_blocks = layout.tokens, layout.seqs, layout.max_blocks
        for name, (offset, size) in layout.sections.items():
            setattr(self, name, device_meta[offset:offset + size])
        if self.n_seqs:       # [groups, sequences, blocks]; a mixer gets its group's table with its view of the cache
            self.block_table = self.block_table.view(layout.groups, self.n_seqs, self.max_blocks)
        self.dtype = dtype
        self.dtype_is_bf16 = dtype == torch.bfloat16
        self.pool = pool
        self.max_count = host_plan.max_count if host_plan is not None else 1
        self.decode = host_plan.decode if host_plan is not None else True
        self.context_limit = host_plan.context_limit if host_plan is not None else SHORT_CONTEXT
        # host-side copies for parts that plan their own work (None while a graph is replayed)
        self.host = host_plan

    def buffer(self, key, rows, cols, dtype):
        return self.pool.take(key, rows, cols, dtype)


class BufferPool:
    """Named workspaces that keep their address from step to step.  A buffer that has to grow is
    replaced, and ``generation`` changes so that captured graphs know their addresses are stale."""

    def __init__(self, device):
        self.device, self.buffers, self.generation, self.frozen = device, {}, 0, False
        self.views = {}         # (key, dtype, rows, cols) -> the view handed out last time: a step asks hundreds of times

    def take(self, key, rows, cols, dtype):
        view = self.views.get((key, dtype, rows, cols))
        if view is not None:
            return view
        asked = dtype
        if isinstance(dtype, str):
            dtype = getattr(torch, dtype)
        need = rows * cols
        held = self.buffers.get((key, dtype))
        if held is None or held.numel() < need:
            if self.frozen:
                raise RuntimeError(f"workspace {key!r} would have to grow while a graph is being captured")
            if held is not None:
                self.generation += 1
                self.views = {k: v for k, v in self.views.items() if k[0] != key}      # they show the old memory
            held = torch.empty(max(need, 1), dtype=dtype, device=self.device)
            self.buffers[(key, dtype)] = held
        view = held[:need].view(rows, cols)
        if len(self.views) > 4096:
            self.views.clear()
        self.views[(key, asked, rows, cols)] = view
        return view

    def bytes(self):
        return sum(t.numel() * t.element_size() for t in self.buffers.values())
