"""The cache on the GPU: paged keys and values for groups of layers, fixed-size state for each
sequence, and the ledger that says who holds what.

Cache entries (one per layer that keeps keys and values, as the model's schedule numbers them)
with the same :class:`KVSpec` form a *group* with storage of its own:
    [entries, blocks, kv_heads, 2, 64 * head_dim]: for each block and head the plane of its keys,
    [64, head_dim], beside the plane of its values, [16, head_dim, 4] (four positions interleaved)
Every group has block lists and a block table of its own: a sequence is equally long in all of
them, but a group that reads only a window of the latest positions gives the blocks behind the
window back while the sequence is still growing.  Fixed-size state ([entries, slots, *shape], zeroed when a slot is handed out) lives beside
it for mixers that carry state instead of, or in addition to, keys and values.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from ..kernels import library as K
from .ledger import BLOCK, CacheLedger


@dataclass(frozen=True)
class KVSpec:
    """What a mixer keeps per token: heads and head size; ``window`` > 0 means that only the last
    ``window`` positions are ever read."""
    kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateSpec:
    """What a mixer keeps per sequence, independent of its length."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


class KVGroup:
    def __init__(self, spec, entries, n_blocks, dtype, device):
        self.spec, self.entries, self.n_blocks = spec, entries, n_blocks
        # Blocks outermost, a block's heads side by side.  The other order (heads outermost, so that
        # the blocks of a prompt are one contiguous run for each head) was measured and lost 3 to 4 %
        # of a decode step at batch 8 and 64, also with the heads' runs skewed by a few blocks: the
        # heads of a sequence are read at the same time and written together, and are then far apart.
        # A head's keys lie beside its values: what a decode step's work-group reads of a block is
        # one run of memory (a per cent at batch 64 against two separate tensors)
        planes = torch.zeros((entries, n_blocks, spec.kv_heads, 2, BLOCK, spec.head_dim), dtype=dtype, device=device)
        self.keys, self.values = planes[:, :, :, 0], planes[:, :, :, 1]
        self.head_stride = 2 * BLOCK * spec.head_dim
        self.block_stride = spec.kv_heads * self.head_stride

    def view(self, entry, block_table, max_blocks):
        """The kernels' view of one entry with the step's block table [n_seqs, max_blocks]."""
        return K.KvView(keys=self.keys[entry].data_ptr(), values=self.values[entry].data_ptr(),
                        blocks=block_table.data_ptr(), max_blocks=max_blocks,
                        kv_heads=self.spec.kv_heads, head_dim=self.spec.head_dim,
                        block_stride=self.block_stride, head_stride=self.head_stride)


class StateGroup:
    def __init__(self, spec, entries, slots, device):
        self.spec, self.entries = spec, entries
        self.data = torch.zeros((entries, slots) + tuple(spec.shape), dtype=getattr(torch, spec.dtype),
                                device=device)


class Cache:
    """``kv_specs[i]`` / ``state_specs[i]`` describe cache entry i (None: the entry keeps none).

    max_tokens  the most tokens live sequences hold together, each sequence rounded up to 64
    max_sequence_length  the longest a single sequence may get (the position encoding's limit)
    """

    def __init__(self, kv_specs, state_specs, max_tokens, max_sequence_length, dtype, device,
                 max_slots=None):
        if max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        n_blocks = (max_tokens + BLOCK - 1) // BLOCK
        self.dtype, self.device = dtype, device
        self.max_tokens = n_blocks * BLOCK
        self.max_sequence_length = min(max_sequence_length, self.max_tokens)
        self.max_blocks = (self.max_sequence_length + BLOCK - 1) // BLOCK
        self.max_slots = max_slots if max_slots is not None else min(n_blocks, 4096)
        self.kv_groups, self.kv_entry = [], {}
        by_spec = {}
        for entry, spec in enumerate(kv_specs):
            if spec is None:
                continue
            by_spec.setdefault(spec, []).append(entry)
        for spec, entries in by_spec.items():
            group = KVGroup(spec, len(entries), n_blocks, dtype, device)
            for index, entry in enumerate(entries):
                self.kv_entry[entry] = (len(self.kv_groups), index)
            self.kv_groups.append(group)
        self.state_groups, self.state_entry = [], {}
        by_spec = {}
        for entry, spec in enumerate(state_specs):
            if spec is None:
                continue
            by_spec.setdefault(spec, []).append(entry)
        for spec, entries in by_spec.items():
            group = StateGroup(spec, len(entries), self.max_slots, device)
            for index, entry in enumerate(entries):
                self.state_entry[entry] = (len(self.state_groups), index)
            self.state_groups.append(group)
        self.ledger = CacheLedger(len(self.kv_groups), n_blocks, self.max_slots, self.max_blocks,
                                  windows=[group.spec.window for group in self.kv_groups])

    # --- slots -----------------------------------------------------------------------------
    def acquire(self):
        slot = self.ledger.acquire()
        for group in self.state_groups:
            group.data[:, slot].zero_()
        return slot

    def release(self, slot):
        self.ledger.release(slot)

    def truncate(self, slot, length):
        """Rewinds a sequence; refused where a mixer keeps state of fixed size, which only ever
        holds the state after the last token (src/cache/tensor/recurrent.rs:3-8)."""
        if self.state_groups and length != self.ledger.lengths[slot]:
            raise ValueError("a model with fixed-size state per sequence cannot be rewound")
        self.ledger.truncate(slot, length)

    def length(self, slot):
        return self.ledger.lengths[slot]

    def blocks(self, slot, group=0):
        """The blocks a sequence holds in one group, by block number (RELEASED where a window has
        moved on)."""
        return self.ledger.held_blocks[group][slot] if self.kv_groups else []

    def block_rows(self, slots):
        """For a step's block tables: [group][sequence] -> block list, a released block's place
        filled with block 0 (a valid block that no kernel reads for this sequence: a query's keys
        start inside its window)."""
        return [[[block if block >= 0 else 0 for block in self.ledger.held_blocks[group][slot]] for slot in slots]
                for group in range(len(self.kv_groups))]

    # --- views -----------------------------------------------------------------------------
    def kv_view(self, entry, block_tables):
        """``block_tables``: the step's tables [groups, n_seqs, max_blocks]."""
        group, index = self.kv_entry[entry]
        return self.kv_groups[group].view(index, block_tables[group], self.max_blocks)

    def state(self, entry):
        """[slots, *shape] state of a cache entry."""
        group, index = self.state_entry[entry]
        return self.state_groups[group].data[index]

    def bytes(self):
        total = sum(g.keys.numel() * g.keys.element_size() * 2 for g in self.kv_groups)
        return total + sum(g.data.numel() * g.data.element_size() for g in self.state_groups)
