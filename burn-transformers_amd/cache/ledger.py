"""Bookkeeping of the cache, without any tensor: which slots are live, how long each sequence
is, and which blocks of each group's storage it holds.

A *slot* is a sequence's handle: its length, its block lists and its row in the per-sequence
state areas.  A *block* holds the keys and values of 64 consecutive positions of one sequence
for every layer of one group; every group has free blocks and block lists of its own.  Slots and
blocks are handed out from free lists and come back when the sequence ends, or earlier where a
group reads only a window of the latest positions; nothing is ever held twice or returned twice
(``check`` proves it).
"""

BLOCK = 64


class CacheFull(RuntimeError):
    """The step needs more slots or blocks than are free.  Nothing was changed."""


class FreeList:
    """Indices 0..n-1; the lowest free index is handed out first."""

    def __init__(self, count):
        self.count = count
        self._free = list(range(count - 1, -1, -1))
        self._held = [False] * count

    def available(self):
        return len(self._free)

    def take(self):
        if not self._free:
            raise CacheFull("no free index")
        index = self._free.pop()
        self._held[index] = True
        return index

    def give(self, index):
        if not (0 <= index < self.count) or not self._held[index]:
            raise ValueError(f"index {index} is not held")
        self._held[index] = False
        self._free.append(index)
        self._free.sort(reverse=True)

    def held(self, index):
        return 0 <= index < self.count and self._held[index]

    def check(self):
        free = set(self._free)
        assert len(free) == len(self._free), "an index is on the free list twice"
        for index in range(self.count):
            assert (index in free) != self._held[index], f"index {index} is neither free nor held, or both"


RELEASED = -1      # in a sequence's block list: a block behind the group's window that went back early


class CacheLedger:
    """``windows[g]`` > 0 says that group g only ever reads the last ``windows[g]`` positions of a
    sequence: its blocks that lie wholly behind that window go back to the free list as soon as the
    sequence has grown past them, and their places in the sequence's list read RELEASED."""

    def __init__(self, n_groups, blocks_per_group, max_slots, max_blocks_per_sequence, windows=None):
        self.n_groups = n_groups
        self.max_blocks_per_sequence = max_blocks_per_sequence
        self.windows = list(windows) if windows is not None else [0] * n_groups
        if len(self.windows) != n_groups or any(w < 0 for w in self.windows):
            raise ValueError(f"{n_groups} groups need {n_groups} windows that are not negative, got {self.windows}")
        self.slots = FreeList(max_slots)
        self.blocks = [FreeList(blocks_per_group) for _ in range(n_groups)]
        self.lengths = [0] * max_slots
        # held_blocks[group][slot][i]: the block that holds positions 64 i .. 64 i + 63 of the sequence
        self.held_blocks = [[[] for _ in range(max_slots)] for _ in range(n_groups)]

    # --- slots -----------------------------------------------------------------------------
    def acquire(self):
        """A fresh slot: length 0, no blocks."""
        try:
            slot = self.slots.take()
        except CacheFull:
            raise CacheFull(f"all {self.slots.count} sequence slots are in use") from None
        self.lengths[slot] = 0
        return slot

    def release(self, slot):
        """Gives the slot and every block it holds back."""
        if not self.slots.held(slot):
            raise ValueError(f"slot {slot} is not live")
        for group in range(self.n_groups):
            for block in self.held_blocks[group][slot]:
                if block != RELEASED:
                    self.blocks[group].give(block)
            self.held_blocks[group][slot] = []
        self.lengths[slot] = 0
        self.slots.give(slot)

    def live(self, slot):
        return self.slots.held(slot)

    def live_slots(self):
        return [slot for slot in range(self.slots.count) if self.slots.held(slot)]

    def first_kept(self, group, length):
        """Number of the first block of a sequence of ``length`` tokens that group ``group`` still
        needs: the next token (position ``length``) reads back to position length - window + 1."""
        window = self.windows[group]
        if window <= 0:
            return 0
        return max(0, length - window + 1) // BLOCK

    def truncate(self, slot, length):
        """Rewinds a live sequence to ``length`` tokens: the blocks it no longer needs go back
        (src/models/llama/model/decode.rs:386-395 rewinds a row the same way; to zero it empties it).
        Refused, before anything changes, where a group with a window has already given back a
        block that the shorter sequence would read again."""
        if not self.slots.held(slot):
            raise ValueError(f"slot {slot} is not live")
        if not (0 <= length <= self.lengths[slot]):
            raise ValueError(f"slot {slot} holds {self.lengths[slot]} tokens and cannot be rewound to {length}")
        keep = self.blocks_for(length)
        for group in range(self.n_groups):
            held = self.held_blocks[group][slot]
            if RELEASED in held[self.first_kept(group, length):keep]:
                raise ValueError(f"slot {slot} cannot be rewound to {length} tokens: a layer with a window of "
                                 f"{self.windows[group]} has given the blocks before it back already")
        for group in range(self.n_groups):
            held = self.held_blocks[group][slot]
            while len(held) > keep:
                block = held.pop()
                if block != RELEASED:
                    self.blocks[group].give(block)
        self.lengths[slot] = length

    # --- growth ----------------------------------------------------------------------------
    @staticmethod
    def blocks_for(length):
        return (length + BLOCK - 1) // BLOCK

    def check_growth(self, new_lengths):
        """Raises unless every slot in {slot: new length} can grow; changes nothing."""
        need = [0] * self.n_groups
        for slot, length in new_lengths.items():
            if not self.slots.held(slot):
                raise ValueError(f"slot {slot} is not live")
            if length < self.lengths[slot]:
                raise ValueError(f"slot {slot} cannot shrink from {self.lengths[slot]} to {length}")
            blocks = self.blocks_for(length)
            if blocks > self.max_blocks_per_sequence:
                raise CacheFull(f"a sequence of {length} tokens needs {blocks} blocks, "
                                f"at most {self.max_blocks_per_sequence} fit one sequence")
            for group in range(self.n_groups):
                need[group] += max(0, blocks - len(self.held_blocks[group][slot]))
        for group in range(self.n_groups):
            if need[group] > self.blocks[group].available():
                raise CacheFull(f"the step needs {need[group]} more blocks of {BLOCK} tokens, "
                                f"{self.blocks[group].available()} are free")

    def reserve(self, slot, length):
        """Makes sure the slot holds blocks for ``length`` positions (the length itself changes
        only at ``commit``).  Returns True if a block was added."""
        added = False
        for group in range(self.n_groups):
            held = self.held_blocks[group][slot]
            while len(held) < self.blocks_for(length):
                held.append(self.blocks[group].take())
                added = True
        return added

    def commit(self, slot, length):
        """The sequence now holds ``length`` tokens; blocks that a group's window has left behind for
        good go back."""
        if length < self.lengths[slot]:
            raise ValueError(f"slot {slot} cannot shrink from {self.lengths[slot]} to {length}")
        self.lengths[slot] = length
        for group in range(self.n_groups):
            if self.windows[group] <= 0:
                continue
            held = self.held_blocks[group][slot]
            for index in range(min(self.first_kept(group, length), len(held))):
                if held[index] != RELEASED:
                    self.blocks[group].give(held[index])
                    held[index] = RELEASED

    # --- proof -----------------------------------------------------------------------------
    def check(self):
        """No slot or block is lost, held twice or free while held; every block a sequence can still
        read is there."""
        self.slots.check()
        for group in range(self.n_groups):
            self.blocks[group].check()
            seen = set()
            for slot in range(self.slots.count):
                held = self.held_blocks[group][slot]
                if not self.slots.held(slot):
                    assert not held and self.lengths[slot] == 0, f"free slot {slot} still holds something"
                needed = self.blocks_for(self.lengths[slot])
                assert len(held) >= needed, f"slot {slot} is longer than its blocks"
                assert RELEASED not in held[self.first_kept(group, self.lengths[slot]):], \
                    f"slot {slot} has given back a block of group {group} that it still reads"
                for block in held:
                    if block == RELEASED:
                        continue
                    assert block not in seen, f"block {block} of group {group} is held twice"
                    assert self.blocks[group].held(block), f"block {block} of group {group} is held but free"
                    seen.add(block)
            assert len(seen) + self.blocks[group].available() == self.blocks[group].count, "a block is lost"
