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
