"""The cache's bookkeeping: no slot or block is lost, held twice or freed twice (no GPU)."""

import random

import pytest

from burn_transformers_amd.cache.ledger import BLOCK, CacheFull, CacheLedger, FreeList


def test_free_list_hands_out_each_index_once():
    pool = FreeList(3)
    taken = [pool.take(), pool.take(), pool.take()]
    assert sorted(taken) == [0, 1, 2] and pool.available() == 0
    with pytest.raises(CacheFull):
        pool.take()
    pool.give(1)
    with pytest.raises(ValueError, match="not held"):
        pool.give(1)                      # freed twice
    with pytest.raises(ValueError, match="not held"):
        pool.give(7)
    assert pool.take() == 1
    pool.check()


def test_growth_is_checked_before_anything_changes():
    ledger = CacheLedger(1, blocks_per_group=4, max_slots=3, max_blocks_per_sequence=3)
    a, b = ledger.acquire(), ledger.acquire()
    ledger.check_growth({a: 100, b: 64})              # 2 + 1 blocks of 4
    with pytest.raises(CacheFull, match="needs 5 more blocks"):
        ledger.check_growth({a: 192, b: 65})
    with pytest.raises(CacheFull, match="at most 3 fit one sequence"):
        ledger.check_growth({a: 193})
    assert ledger.blocks[0].available() == 4 and ledger.lengths[a] == 0
    ledger.reserve(a, 100)
    ledger.commit(a, 100)
    assert len(ledger.held_blocks[0][a]) == 2
    assert not ledger.reserve(a, 128) and ledger.reserve(a, 129)
    with pytest.raises(ValueError, match="cannot shrink"):
        ledger.commit(a, 50)
    with pytest.raises(ValueError, match="not live"):
        ledger.check_growth({2: 5})
    ledger.release(a)
    with pytest.raises(ValueError, match="not live"):
        ledger.release(a)                 # released twice
    ledger.check()
    assert ledger.blocks[0].available() == 4


def test_slots_and_blocks_are_used_again():
    ledger = CacheLedger(1, blocks_per_group=6, max_slots=2, max_blocks_per_sequence=6)
    first = ledger.acquire()
    ledger.reserve(first, 130)
    ledger.commit(first, 130)
    blocks = list(ledger.held_blocks[0][first])
    with pytest.raises(CacheFull, match="slots"):
        ledger.acquire(), ledger.acquire()
    ledger.release(first)
    ledger.release(1)
    again = ledger.acquire()
    assert again == first and ledger.lengths[again] == 0 and not ledger.held_blocks[0][again]
    ledger.reserve(again, 64 * 3)
    assert set(ledger.held_blocks[0][again]) == set(blocks)
    ledger.check()


def test_random_traffic_keeps_the_invariants():
    rng = random.Random(0)
    ledger = CacheLedger(1, blocks_per_group=40, max_slots=12, max_blocks_per_sequence=8)
    live = {}
    for _ in range(3000):
        action = rng.random()
        if action < 0.25 and ledger.slots.available():
            live[ledger.acquire()] = 0
        elif action < 0.45 and live:
            slot = rng.choice(list(live))
            ledger.release(slot)
            del live[slot]
        elif live:
            grow = {s: live[s] + rng.randint(1, 90) for s in rng.sample(list(live), rng.randint(1, len(live)))}
            try:
                ledger.check_growth(grow)
            except CacheFull:
                continue
            for slot, length in grow.items():
                ledger.reserve(slot, length)
                ledger.commit(slot, length)
                live[slot] = length
        ledger.check()
        held = sum(len(ledger.held_blocks[0][s]) for s in live)
        assert held + ledger.blocks[0].available() == 40
        assert all(len(ledger.held_blocks[0][s]) == (n + BLOCK - 1) // BLOCK for s, n in live.items())
    for slot in list(live):
        ledger.release(slot)
    ledger.check()
    assert ledger.blocks[0].available() == 40 and ledger.slots.available() == 12


def test_truncate_gives_blocks_back_and_keeps_the_rest():
    ledger = CacheLedger(1, 8, 4, 8)
    a, b = ledger.acquire(), ledger.acquire()
    for slot, length in ((a, 200), (b, 70)):
        ledger.check_growth({slot: length})
        ledger.reserve(slot, length)
        ledger.commit(slot, length)
    assert ledger.blocks[0].available() == 8 - 4 - 2
    kept = list(ledger.held_blocks[0][a][:2])
    ledger.truncate(a, 65)                      # 65 tokens need two of the four blocks
    assert ledger.lengths[a] == 65 and ledger.held_blocks[0][a] == kept
    assert ledger.blocks[0].available() == 8 - 2 - 2
    ledger.check()
    ledger.truncate(a, 0)                       # to zero: the slot stays live and holds nothing
    assert ledger.live(a) and ledger.held_blocks[0][a] == [] and ledger.live_slots() == [a, b]
    with pytest.raises(ValueError, match="cannot be rewound to 71"):
        ledger.truncate(b, 71)
    with pytest.raises(ValueError, match="not live"):
        ledger.truncate(3, 0)
    ledger.check_growth({a: 130})
    ledger.reserve(a, 130)
    ledger.commit(a, 130)
    ledger.check()


def test_a_group_with_a_window_gives_blocks_back_while_the_sequence_grows():
    """Two groups: one keeps every key, one reads only the last 100 positions.  The second gives a
    block back as soon as the next token can no longer read any of its positions; the first keeps
    all; both have free lists of their own."""
    from burn_transformers_amd.cache.ledger import RELEASED
    ledger = CacheLedger(2, blocks_per_group=8, max_slots=2, max_blocks_per_sequence=8, windows=[0, 100])
    a = ledger.acquire()
    length = 0
    for grow in (60, 70, 40, 1, 1, 90, 150, 30):
        length += grow
        ledger.check_growth({a: length})
        ledger.reserve(a, length)
        ledger.commit(a, length)
        ledger.check()
        blocks = (length + BLOCK - 1) // BLOCK
        first = max(0, length - 100 + 1) // BLOCK           # the block of the oldest position the next token reads
        full, windowed = ledger.held_blocks[0][a], ledger.held_blocks[1][a]
        assert len(full) == blocks and RELEASED not in full
        assert windowed[:first] == [RELEASED] * first and RELEASED not in windowed[first:] and len(windowed) == blocks
        assert ledger.blocks[0].available() == 8 - blocks and ledger.blocks[1].available() == 8 - (blocks - first)
    assert length == 442 and ledger.blocks[1].available() == 6      # 7 blocks long, 2 of them still held
    # a second sequence can use what the window gave back, though the first group is nearly full
    b = ledger.acquire()
    with pytest.raises(CacheFull, match="needs 2 more blocks"):
        ledger.check_growth({b: 100})                      # the group that keeps everything has one block left
    ledger.check_growth({b: 64})
    ledger.reserve(b, 64)
    ledger.commit(b, 64)
    ledger.check()
    # rewinding: fine while the shorter sequence reads nothing that is gone, refused otherwise, and
    # a refusal changes nothing
    before = ([list(x) for x in ledger.held_blocks[0]], [list(x) for x in ledger.held_blocks[1]], list(ledger.lengths))
    with pytest.raises(ValueError, match="window of 100 has given the blocks before it back"):
        ledger.truncate(a, 300)
    assert ([list(x) for x in ledger.held_blocks[0]], [list(x) for x in ledger.held_blocks[1]], list(ledger.lengths)) == before
    ledger.truncate(a, 420)                                 # reads back to 321: block 5, which is still there
    assert ledger.lengths[a] == 420 and len(ledger.held_blocks[1][a]) == 7
    ledger.check()
    ledger.release(a)
    ledger.release(b)
    ledger.check()
    assert [f.available() for f in ledger.blocks] == [8, 8]


def test_random_traffic_with_windows_keeps_the_books():
    rng = random.Random(7)
    ledger = CacheLedger(3, blocks_per_group=30, max_slots=6, max_blocks_per_sequence=10, windows=[0, 64, 200])
    live = {}
    for _ in range(600):
        action = rng.random()
        if action < 0.2 and ledger.slots.available():
            live[ledger.acquire()] = 0
        elif action < 0.3 and live:
            slot = rng.choice(list(live))
            ledger.release(slot)
            del live[slot]
        elif live:
            slot = rng.choice(list(live))
            target = min(live[slot] + rng.randint(1, 150), 640)
            try:
                ledger.check_growth({slot: target})
            except CacheFull:
                continue
            ledger.reserve(slot, target)
            if rng.random() < 0.1:                          # a pass that failed: the reservation is undone
                ledger.truncate(slot, live[slot])
            else:
                ledger.commit(slot, target)
                live[slot] = target
        ledger.check()
    for slot in list(live):
        ledger.release(slot)
    ledger.check()
    assert all(f.available() == 30 for f in ledger.blocks)
