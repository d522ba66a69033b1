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


def token_capacity(tokens):
    """The class of a step by its tokens: steps of up to 64 tokens are their own class; beyond, the
    classes are 65 .. 128, 129 .. 192 and so on.  Every step of a class lays its tables out for the
    class's most tokens and reserves its workspaces for them, and every choice of kernels that the
    parts make by a step's rows is the same for a whole class (they turn at 64, 128 and 256 rows), so
    that one launch list serves the class: only the counts in its calls differ from step to step."""
    return tokens if tokens <= BLOCK else (tokens + BLOCK - 1) // BLOCK * BLOCK


class StepLayout:
    """Offsets of the sections for T tokens, B sequences, R wanted rows.  The sections that hold one
    word per token have room for the step's class (``token_capacity``), so that the later sections
    start at the same place in every step of a class."""

    def __init__(self, tokens, seqs, rows, max_blocks, groups=1):
        self.tokens, self.seqs, self.rows, self.max_blocks, self.groups = tokens, seqs, rows, max_blocks, groups
        self.capacity = token_capacity(tokens)
        offset = 0
        self.sections = {}
        for name, size, room in (("tok_ids", tokens, self.capacity), ("tok_pos", tokens, self.capacity),
                                 ("tok_seq", tokens, self.capacity),
                                 ("seq_off", seqs + 1, seqs + 1), ("seq_start", seqs, seqs), ("slots", seqs, seqs),
                                 ("sel_rows", rows, rows), ("block_table", groups * seqs * max_blocks, groups * seqs * max_blocks)):
            self.sections[name] = (offset, size)
            offset = _align(offset + room)
        self.total = offset

    def key(self):
        return (self.tokens, self.seqs, self.rows, self.max_blocks, self.groups)

    def class_key(self):
        """What the steps that one launch list serves have in common."""
        return (self.capacity, self.seqs, self.rows, self.max_blocks, self.groups)


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
        self.token_capacity = layout.capacity        # most tokens of a step of this class: workspaces are reserved for them
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
        """A workspace [rows, cols] that keeps its address from step to step.  One that holds a row
        (or several) per token of the step is reserved for the most tokens of the step's class, so
        that it stays where it is for every step of the class."""
        reserve = rows
        if self.n_tokens and self.token_capacity != self.n_tokens and rows % self.n_tokens == 0:
            reserve = rows // self.n_tokens * self.token_capacity
        return self.pool.take(key, rows, cols, dtype, reserve)

    def partial_sums(self, key, splits, rows, cols):
        """float32 [splits, rows, cols] for the slices of a product whose K range is cut, the slices
        as far apart as the step's class needs: the same distance in every step of the class."""
        room = self.token_capacity if rows == self.n_tokens else rows
        return self.buffer(key, splits * room, cols, "float32").view(splits, room, cols)[:, :rows]


class BufferPool:
    """Named workspaces that keep their address from step to step.  A buffer that has to grow is
    replaced, and ``generation`` changes so that captured graphs know their addresses are stale."""

    def __init__(self, device):
        self.device, self.buffers, self.generation, self.frozen = device, {}, 0, False
        self.views = {}         # (key, dtype, rows, cols) -> the view handed out last time: a step asks hundreds of times

    def take(self, key, rows, cols, dtype, reserve_rows=0):
        """``reserve_rows``: rows to make room for where the workspace has to be made or replaced."""
        view = self.views.get((key, dtype, rows, cols))
        if view is not None:
            return view
        asked = dtype
        if isinstance(dtype, str):
            dtype = getattr(torch, dtype)
        need = rows * cols
        held = self.buffers.get((key, dtype))
        if held is None or held.numel() < need:
            need = max(need, reserve_rows * cols)
            if self.frozen:
                raise RuntimeError(f"workspace {key!r} would have to grow while a graph is being captured")
            if held is not None:
                self.generation += 1
                self.views = {k: v for k, v in self.views.items() if k[0] != key}      # they show the old memory
            held = torch.empty(max(need, 1), dtype=dtype, device=self.device)
            self.buffers[(key, dtype)] = held
        view = held[:rows * cols].view(rows, cols)
        if len(self.views) > 4096:
            self.views.clear()
        self.views[(key, asked, rows, cols)] = view
        return view

    def bytes(self):
        return sum(t.numel() * t.element_size() for t in self.buffers.values())
