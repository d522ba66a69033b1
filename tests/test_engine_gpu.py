"""The engine against the plain implementation: every way of cutting and batching the same
requests gives the same logits, in float32 and in bfloat16."""

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from model_helpers import CONFIGS, model_folder, plain_logits, prompts_for, tolerance  # noqa: E402

DTYPES = ["float32", "bfloat16"]
_models = {}


def engine_for(name, dtype, max_tokens=2048, gain=1.0, **kw):
    # these tests are about what graphs replay: every repeating shape is captured, also where the
    # engine's own choice (graphs=True: only where a graph pays) would leave a shape to its list
    kw["graphs"] = "always" if kw.get("graphs", True) else False
    key = (name, dtype, gain)
    if key not in _models:
        folder, _, _ = model_folder(name, gain)
        _models[key] = bt.load_model(folder, dtype=dtype, device="cuda:0")
    return bt.Engine(_models[key], max_tokens=max_tokens, **kw)


def check(got, want, dtype, what):
    got = got.detach().cpu().double()
    err = float((got - want).abs().max())
    assert torch.isfinite(got).all(), what
    assert err <= tolerance(dtype, want), f"{what}: max abs error {err} > {tolerance(dtype, want)}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", [("A", [5, 11, 17, 100]), ("B", [1, 23, 64]), ("BW", [64, 65, 150]), ("C", [3, 80])])
def test_each_request_alone_and_whole(name, dtype, lengths):
    engine = engine_for(name, dtype)
    for ids in prompts_for(name, lengths):
        slot = engine.open()
        logits = engine.step([(slot, ids)], want=[list(range(len(ids)))])
        check(logits, plain_logits(name, ids), dtype, f"{name} whole {len(ids)}")
        engine.close(slot)
    engine.cache.ledger.check()


@pytest.mark.parametrize("name,lengths", [("A", [100, 66]), ("BW", [150])])
def test_prompts_without_the_vendor_library(name, lengths, monkeypatch):
    """Prompts of more than 64 tokens on the package's own tile kernel and fused cache scatter."""
    from burn_transformers_amd.kernels import library as K
    monkeypatch.setitem(K._library_state, "tried", True)
    monkeypatch.setitem(K._library_state, "lib", None)
    engine = engine_for(name, "bfloat16")
    prompts = prompts_for(name, lengths, seed=5)
    slots = [engine.open() for _ in prompts]
    logits = engine.step(list(zip(slots, prompts)), want=[list(range(len(p))) for p in prompts])
    begin = 0
    for ids in prompts:
        check(logits[begin:begin + len(ids)], plain_logits(name, ids), "bfloat16", f"{name} own kernels {len(ids)}")
        begin += len(ids)
    step = engine.step([(slot, [7]) for slot in slots])      # the cache the scatter filled is read
    for row, ids in enumerate(prompts):
        check(step[row:row + 1], plain_logits(name, ids + [7])[-1:], "bfloat16", f"{name} own kernels, next token")
    for slot in slots:
        engine.close(slot)


def test_a_step_of_many_thousand_prompt_tokens():
    """70 prompts of up to 128 tokens in one step: more rows than one call of the vendor's library
    is given, and more sequences than a decode batch of the measured sizes."""
    name = "A"
    engine = engine_for(name, "bfloat16", max_tokens=70 * 128)
    lengths = [128 - (i % 5) for i in range(70)]
    prompts = prompts_for(name, lengths, seed=8)
    assert sum(lengths) > 2 * 4096
    slots = [engine.open() for _ in prompts]
    logits = engine.step(list(zip(slots, prompts)), want=[[0, n - 1] for n in lengths]).clone()
    for i in (0, 1, 33, 34, 68, 69):           # requests at both ends and across the runs of rows
        check(logits[2 * i:2 * i + 2], plain_logits(name, prompts[i])[[0, lengths[i] - 1]], "bfloat16", f"request {i}")
    for slot in slots:
        engine.close(slot)
    engine.cache.ledger.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,length", [("A", 100), ("BW", 150), ("B", 33), ("B", 64), ("C", 70)])
def test_last_32_tokens_one_by_one(name, dtype, length):
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [length], seed=3)[0]
    want = plain_logits(name, ids)
    slot = engine.open()
    head = length - 32
    rows = []
    if head > 0:
        rows.append(engine.step([(slot, ids[:head])], want=[list(range(head))]).clone())
    for t in range(max(head, 0), length):
        rows.append(engine.step([(slot, [ids[t]])]).clone())
    check(torch.cat(rows), want, dtype, f"{name} decode tail of {length}")
    assert engine.graph_replays > 0
    engine.close(slot)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(name, dtype):
    """Token by token from the very first token."""
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [20], seed=4)[0]
    slot = engine.open()
    rows = [engine.step([(slot, [t])]).clone() for t in ids]
    check(torch.cat(rows), plain_logits(name, ids), dtype, f"{name} from the first token")
    engine.close(slot)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,chunk,lengths", [("A", 7, [1, 23, 40]), ("BW", 64, [150, 70, 3]), ("B", 7, [1, 23]), ("B", 5, [9])])
def test_chunked_prompts(name, dtype, chunk, lengths):
    engine = engine_for(name, dtype)
    prompts = prompts_for(name, lengths, seed=5)
    slots = [engine.open() for _ in prompts]
    got = [[] for _ in prompts]
    for begin in range(0, max(lengths), chunk):
        rows = [i for i, p in enumerate(prompts) if len(p) > begin]
        entries = [(slots[i], prompts[i][begin:begin + chunk]) for i in rows]
        want = [list(range(len(e[1]))) for e in entries]
        logits = engine.step(entries, want).clone()
        at = 0
        for i, e in zip(rows, entries):
            got[i].append(logits[at:at + len(e[1])])
            at += len(e[1])
    for i, p in enumerate(prompts):
        check(torch.cat(got[i]), plain_logits(name, p), dtype, f"{name} chunks of {chunk}, prompt {i}")
    for s in slots:
        engine.close(s)
    engine.cache.ledger.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "BW"])
def test_unequal_batches_one_after_another(name, dtype):
    """Batches of unequal prompts, decoded with teacher forcing; shorter requests end earlier and
    their slots are used again by the next batch, whose results must not see the old occupants."""
    limit = CONFIGS[name][0]["n_positions"]
    engine = engine_for(name, dtype, max_tokens=64 * 8)
    batches = [[5, 70, 17], [64, 3, 90, 1], [33, 33], [100, 2, 65]]
    seen_slots = []
    for b, lengths in enumerate(batches):
        totals = [min(n + 9 + 5 * i, limit) for i, n in enumerate(lengths)]
        requests = prompts_for(name, totals, seed=10 + b)
        slots = [engine.open() for _ in requests]
        seen_slots.append(list(slots))
        got = [[] for _ in requests]
        logits = engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, lengths)],
                             want=[list(range(n)) for n in lengths]).clone()
        at = 0
        for i, n in enumerate(lengths):
            got[i].append(logits[at:at + n])
            at += n
        live = list(range(len(requests)))
        position = list(lengths)
        while live:
            entries = [(slots[i], [requests[i][position[i]]]) for i in live]
            logits = engine.step(entries).clone()
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                position[i] += 1
            for i in [i for i in live if position[i] >= totals[i]]:
                engine.close(slots[i])            # ends earlier than the others
                live.remove(i)
        for i, r in enumerate(requests):
            check(torch.cat(got[i]), plain_logits(name, r), dtype, f"{name} batch {b} request {i}")
        engine.cache.ledger.check()
    assert set(seen_slots[0]) & set(seen_slots[1]), "slots were not used again"
    assert engine.cache.ledger.slots.available() == engine.cache.max_slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,count", [("A", 16), ("BW", 17), ("A", 40), ("BW", 64), ("A", 70)])
def test_wide_decode_batches(name, dtype, count):
    """Decode steps of 16, 17..64 and more than 64 sequences take other kernels than small batches do."""
    engine = engine_for(name, dtype, max_tokens=64 * count)
    lengths = [3 + (7 * i) % 20 for i in range(count)]
    requests = prompts_for(name, [n + 3 for n in lengths], seed=70)
    slots = [engine.open() for _ in requests]
    for begin in range(0, count, 8):
        part = range(begin, min(begin + 8, count))
        engine.step([(slots[i], requests[i][:lengths[i]]) for i in part], want=[[] for _ in part])
    got = []
    for t in range(3):
        got.append(engine.step([(s, [r[n + t]]) for s, r, n in zip(slots, requests, lengths)]).clone())
    for i in (0, 1, count // 2, count - 1):
        want = plain_logits(name, requests[i])[lengths[i]:]
        check(torch.stack([g[i] for g in got]), want, dtype, f"{name} sequence {i} of {count}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "BW", "C"])
def test_decoding_from_packed_weight_copies_changes_no_bit(name, dtype):
    """Decode steps read second copies of the layers' matrices, packed for the skinny kernel; with
    the copies switched off the same steps read the plain matrices and give the same bits."""
    from burn_transformers_amd.kernels import library as K
    runs = []
    for enabled in (True, False):
        K.PackedWeight.enabled = enabled
        try:
            engine = engine_for(name, dtype, graphs=False)
            requests = prompts_for(name, [9, 1, 30, 17, 5], seed=11)
            slots = [engine.open() for _ in requests]
            rows = [engine.step(list(zip(slots, requests))).clone()]
            for _ in range(6):
                ids = rows[-1].argmax(-1).tolist()
                rows.append(engine.step([(s, [t]) for s, t in zip(slots, ids)]).clone())
            runs.append(torch.stack(rows))
        finally:
            K.PackedWeight.enabled = True
    assert torch.equal(runs[0], runs[1])
    mixer = engine.model.blocks[0].parts["mixer"]
    assert mixer.qkv_packed is not None and mixer.qkv_packed.for_step(5, 1) is not None     # the copies were in use


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,count", [("A", 17), ("BW", 33), ("C", 40), ("BW", 64)])
def test_chunk_major_activations_change_no_bit(name, count, dtype):
    """In decode steps of up to 64 sequences the activations between the kernels are kept chunk-major
    (the layout the skinny product reads fastest); with that switched off the same steps give the
    same bits."""
    from burn_transformers_amd.kernels import library as K
    runs = []
    for enabled in (True, False):
        K.Chunked.enabled = enabled
        try:
            engine = engine_for(name, dtype, max_tokens=64 * (count + 1), graphs=False)
            requests = prompts_for(name, [2 + (5 * i) % 9 for i in range(count)], seed=33)
            slots = [engine.open() for _ in requests]
            rows = []
            for begin in range(0, count, 8):
                part = range(begin, min(begin + 8, count))
                rows.append(engine.step([(slots[i], requests[i]) for i in part]).clone())
            logits = torch.cat(rows)
            rows = [logits]
            for _ in range(4):
                ids = rows[-1].argmax(-1).tolist()
                rows.append(engine.step([(s, [t]) for s, t in zip(slots, ids)]).clone())
            # prompts of 17 to 64 tokens: the norms and the feed-forward use the layout there too
            for length in (17, 40, 64):
                slot = engine.open()
                ids = prompts_for(name, [length], seed=length)[0]
                rows.append(engine.step([(slot, ids)], want=[[0, length - 1]]).sum(0, keepdim=True).expand(count, -1).clone())
                engine.close(slot)
            runs.append(torch.stack(rows))
        finally:
            K.Chunked.enabled = True
    assert torch.equal(runs[0], runs[1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_reused_blocks_do_not_leak(dtype):
    """A slot's blocks are poisoned with NaN after it is closed; the next occupant must not care."""
    engine = engine_for("A", dtype, max_tokens=256)
    first = prompts_for("A", [120], seed=20)[0]
    slot = engine.open()
    engine.step([(slot, first)])
    engine.close(slot)
    for group in engine.cache.kv_groups:
        group.keys.fill_(float("nan"))
        group.values.fill_(float("nan"))
    ids = prompts_for("A", [50], seed=21)[0]
    slot = engine.open()
    rows = [engine.step([(slot, ids[:30])], want=[list(range(30))]).clone()]
    rows += [engine.step([(slot, [t])]).clone() for t in ids[30:]]
    check(torch.cat(rows), plain_logits("A", ids), dtype, "poisoned cache")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype):
    """Decoding far past several block edges, against whole-sequence logits."""
    engine = engine_for("BW", dtype)
    ids = prompts_for("BW", [192], seed=30)[0]
    want = plain_logits("BW", ids)
    slot = engine.open()
    rows = [engine.step([(slot, ids[:2])], want=[[0, 1]]).clone()]
    rows += [engine.step([(slot, [t])]).clone() for t in ids[2:]]
    check(torch.cat(rows), want, dtype, "long decode")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_over_contexts_of_thousands(dtype):
    """With contexts this long a decode step cuts every sequence's keys into runs for separate
    work-groups (a short sequence beside the long ones has empty runs); the steps come from graphs
    of their own class of context, and crossing 4,096 tokens starts the next class."""
    engine = engine_for("L", dtype, max_tokens=4352 + 2112 + 64, gain=2.0)
    requests = prompts_for("L", [4110, 2070, 40], seed=33)
    want = [plain_logits("L", r, 2.0) for r in requests]
    decoded = 22
    slots = [engine.open() for _ in requests]
    rows = [[engine.step([(slot, r[:-decoded])]).clone()] for slot, r in zip(slots, requests)]
    assert ("attention.partial", torch.float32) not in engine.pool.buffers
    for i in range(decoded, 0, -1):
        logits = engine.step([(slot, [r[-i]]) for slot, r in zip(slots, requests)])
        for row, got in zip(rows, logits):
            row.append(got[None].clone())
    assert ("attention.partial", torch.float32) in engine.pool.buffers and engine.graph_replays >= decoded - 4
    for r, got, full in zip(requests, rows, want):
        check(torch.cat(got), full[len(r) - decoded - 1:], dtype, f"request of {len(r)} tokens")


def test_graph_and_eager_decoding_agree_bitwise():
    ids = prompts_for("A", [40], seed=31)[0]
    outs = []
    for graphs in (True, False):
        engine = engine_for("A", "bfloat16", graphs=graphs)
        slot = engine.open()
        rows = [engine.step([(slot, ids[:8])]).clone()]
        rows += [engine.step([(slot, [t])]).clone() for t in ids[8:]]
        outs.append(torch.cat(rows))
        assert (engine.graph_replays > 0) == graphs
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,chunk", [("A", 40), ("BW", 70)])
def test_prompt_steps_of_a_repeating_shape_are_replayed_from_graphs(name, dtype, chunk):
    """Chunks of prompts whose shape repeats (same counts; other ids, positions, slots and wanted
    places) run from a graph from the third time on, with the engine's eager steps and waits for the
    device between the replays; every replay is bitwise what an engine without graphs computes."""
    replayed = engine_for(name, dtype, max_tokens=64 * 8)
    plain_engine = engine_for(name, dtype, max_tokens=64 * 8, graphs=False)
    counts = [chunk, chunk - 9, 3]
    replays_of_prompts = 0
    for rep in range(4):
        requests = prompts_for(name, [2 * c + 2 for c in counts], seed=50 + rep)
        slots = [(replayed.open(), plain_engine.open()) for _ in requests]
        if rep % 2:                         # other slots and blocks than last time
            extra = (replayed.open(), plain_engine.open())
        for part in range(2):               # two steps of the same shape, the second on a filled cache
            want = [[(rep + part) % c, c - 1] for c in counts] if part else [[] for _ in counts]
            entries = lambda which: [(s[which], r[part * c:(part + 1) * c]) for s, r, c in zip(slots, requests, counts)]
            before = replayed.graph_replays
            got = replayed.step(entries(0), want).clone()
            replays_of_prompts += replayed.graph_replays - before
            torch.cuda.synchronize()
            assert torch.equal(got, plain_engine.step(entries(1), want)), (rep, part)
        for t in range(2):                  # single tokens in between: graphs of their own
            entries = lambda which: [(s[which], [r[2 * c + t]]) for s, r, c in zip(slots, requests, counts)]
            assert torch.equal(replayed.step(entries(0)).clone(), plain_engine.step(entries(1)))
        if rep == 3:
            rows = [2 * c - 1 for c in counts]
            for (slot, _), request, row in zip(slots, requests, rows):
                assert replayed.length(slot) == len(request)
        for pair in slots + ([extra] if rep % 2 else []):
            replayed.close(pair[0])
            plain_engine.close(pair[1])
    assert replays_of_prompts >= 3          # each kind of step came four times: twice eagerly, then captured and replayed
    replayed.cache.ledger.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_schedule_with_and_without_graphs(dtype):
    """A hundred steps of random shape from a small set (so that shapes repeat and are replayed from
    graphs), sequences that end and slots that are used again: the engine with graphs and the one
    without give the same bits at every step, and the last logits of every sequence are the plain
    implementation's."""
    import random
    name = "BW"
    limit = CONFIGS[name][0]["n_positions"]
    replayed = engine_for(name, dtype, max_tokens=64 * 12)
    eager = engine_for(name, dtype, max_tokens=64 * 12, graphs=False)
    rng = random.Random(7)
    live = {}                                   # request number -> dict(slots, tokens, fed)
    next_request = 0
    for step_number in range(100):
        while len(live) < 4 and (len(live) < 2 or rng.random() < 0.3):
            tokens = prompts_for(name, [rng.choice([30, 64, 100, 150])], seed=100 + next_request)[0]
            live[next_request] = dict(slots=(replayed.open(), eager.open()), tokens=tokens, fed=0)
            next_request += 1
        chosen = [r for r in live if rng.random() < 0.9] or list(live)
        width = rng.choice([1, 1, 1, 7, 33])            # most steps bring one token per sequence
        counts = {r: min(width if rng.random() < 0.9 else 2, len(live[r]["tokens"]) - live[r]["fed"]) for r in chosen}
        entries = lambda which: [(live[r]["slots"][which], live[r]["tokens"][live[r]["fed"]:live[r]["fed"] + counts[r]])
                                 for r in chosen]
        want = [[counts[r] - 1] if rng.random() < 0.8 else [] for r in chosen]
        got = replayed.step(entries(0), want).clone()
        assert torch.equal(got, eager.step(entries(1), want)), f"step {step_number}"
        row = 0
        for r, places in zip(chosen, want):
            live[r]["fed"] += counts[r]
            if places:
                if live[r]["fed"] == len(live[r]["tokens"]):
                    check(got[row:row + 1], plain_logits(name, live[r]["tokens"])[-1:], dtype, f"request {r}")
                row += 1
            if live[r]["fed"] == len(live[r]["tokens"]):
                replayed.close(live[r]["slots"][0])
                eager.close(live[r]["slots"][1])
                del live[r]
        replayed.cache.ledger.check()
    assert replayed.graph_replays > 10, replayed.graph_replays


@pytest.mark.parametrize("dtype", DTYPES)
def test_rewound_sequences_go_on_as_if_the_rest_had_never_been(dtype):
    """truncate() rewinds a sequence (the blocks it no longer needs go back), other tokens are fed
    from there, and the logits are those of the new sequence; reset() ends everything."""
    name = "BW"
    engine = engine_for(name, dtype, max_tokens=64 * 6)
    first, second = prompts_for(name, [150, 100], seed=61)
    a, b = engine.open(), engine.open()
    engine.step([(a, first), (b, second)])
    free_before = engine.cache.ledger.blocks[0].available()
    engine.truncate(a, 70)                                  # 150 -> 70 tokens: one of three blocks goes back
    assert engine.length(a) == 70 and engine.cache.ledger.blocks[0].available() == free_before + 1
    other = prompts_for(name, [40], seed=62)[0]
    logits = engine.step([(a, other), (b, [5])], want=[list(range(40)), [0]])
    check(logits[:40], plain_logits(name, first[:70] + other)[70:], dtype, "after the rewind")
    check(logits[40:], plain_logits(name, second + [5])[-1:], dtype, "the other sequence")
    engine.truncate(a, 0)                                   # to nothing: the slot stays open
    logits = engine.step([(a, other[:9])], want=[[8]])
    check(logits, plain_logits(name, other[:9])[-1:], dtype, "from the start again")
    with pytest.raises(ValueError, match="cannot be rewound"):
        engine.truncate(a, 10)
    engine.cache.ledger.check()
    engine.reset()
    assert engine.cache.ledger.live_slots() == [] and \
        engine.cache.ledger.blocks[0].available() == engine.cache.ledger.blocks[0].count
    engine.cache.ledger.check()


def test_refused_steps_change_nothing():
    engine = engine_for("A", "float32", max_tokens=128)
    slot = engine.open()
    engine.step([(slot, [1, 2, 3])])
    before = (engine.length(slot), list(engine.cache.blocks(slot)))
    from burn_transformers_amd.engine.engine import StepError
    with pytest.raises(StepError, match="token values in 0..1000"):
        engine.step([(slot, [5, 1000])])
    with pytest.raises(StepError, match="outside its"):
        engine.step([(slot, [5])], want=[[1]])
    with pytest.raises(StepError, match="limit"):
        engine.step([(slot, [1] * 126)])
    with pytest.raises(StepError, match="twice"):
        engine.step([(slot, [1]), (slot, [2])])
    with pytest.raises(StepError, match="expected integers"):
        engine.step([(slot, [1.9, 2.0])])
    other = engine.open()
    with pytest.raises(StepError, match="blocks"):
        engine.step([(other, [1] * 100)])          # 2 blocks needed, 1 free
    assert (engine.length(slot), list(engine.cache.blocks(slot))) == before
    assert engine.length(other) == 0 and not engine.cache.blocks(other)
    engine.cache.ledger.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_idle_entries_run_nothing_commit_nothing_and_read_as_zeros(dtype):
    """An entry without tokens is a no-op with exact zero logits, and a step of nothing but such
    entries commits nothing (src/models/llama/model/decode.rs:43-44, 648-650, 730-751; the
    reference's test is decode_tests.rs:382): lengths, blocks and the steps counted stay, and the
    entries beside an idle one get the logits they get without it, bit for bit."""
    from burn_transformers_amd.engine.engine import StepError
    name = "A"
    engine = engine_for(name, dtype, graphs=False)
    first, second, third = prompts_for(name, [20, 9, 70], seed=31)
    a, b, c = engine.open(), engine.open(), engine.open()
    engine.step([(a, first[:10]), (b, second[:8]), (c, third[:64])])
    ledger = engine.cache.ledger
    before = (list(ledger.lengths), [list(x) for x in ledger.held_blocks[0]], ledger.blocks[0].available(), engine.steps_run)
    state = lambda: (list(ledger.lengths), [list(x) for x in ledger.held_blocks[0]], ledger.blocks[0].available(), engine.steps_run)
    vocab = CONFIGS[name][0]["vocab_size"]
    # nothing at all, and nothing but idle entries, with and without wanted places
    assert tuple(engine.step([]).shape) == (0, vocab)
    zeros = engine.step([(a, []), (b, []), (c, [])])
    assert tuple(zeros.shape) == (3, vocab) and zeros.dtype == torch.float32 and not zeros.any()
    assert tuple(engine.step([(a, []), (c, [])], want=[[], []]).shape) == (0, vocab)
    assert state() == before
    with pytest.raises(StepError, match="outside its 0 tokens"):
        engine.step([(a, []), (b, [second[8]])], want=[[0], [0]])
    assert state() == before
    # an idle entry between two that go on: its row is zeros, theirs are what they are without it
    mixed = engine.step([(a, [first[10]]), (b, []), (c, third[64:])]).clone()
    assert not mixed[1].any()
    assert [engine.length(s) for s in (a, b, c)] == [11, 8, 70]
    check(mixed[0:1], plain_logits(name, first[:11])[-1:], dtype, "beside an idle entry, decode row")
    check(mixed[2:3], plain_logits(name, third)[-1:], dtype, "beside an idle entry, prompt row")
    engine.truncate(a, 10)
    engine.truncate(c, 64)
    alone = engine.step([(a, [first[10]]), (c, third[64:])])
    assert torch.equal(alone[0], mixed[0]) and torch.equal(alone[1], mixed[2])
    # wanted places given: the idle entry has none, and takes no row
    some = engine.step([(a, [first[11]]), (b, []), (c, [])], want=[[0], [], []])
    assert tuple(some.shape) == (1, vocab)
    check(some, plain_logits(name, first[:12])[-1:], dtype, "explicit places beside idle entries")
    # the idle sequence goes on afterwards as if nothing had been
    check(engine.step([(b, [second[8]])]), plain_logits(name, second)[-1:], dtype, "after idling")
    ledger.check()
    engine.reset()


@pytest.mark.parametrize("graphs", [False, True])
def test_tokens_that_are_on_the_gpu_already_feed_a_step_from_there(graphs):
    """``device_tokens``: the step reads its tokens from a tensor on the GPU (what a selection has
    just chosen) instead of from the entries; same logits, bit for bit, as the same tokens given
    by the host, also when the step is replayed from a graph."""
    from burn_transformers_amd.engine.engine import StepError
    name = "A"
    by_host, by_device = engine_for(name, "bfloat16", graphs=graphs), engine_for(name, "bfloat16", graphs=graphs)
    requests = prompts_for(name, [30, 9, 50], seed=90)
    slots_h = [by_host.open() for _ in requests]
    slots_d = [by_device.open() for _ in requests]
    by_host.step([(s, r[:5]) for s, r in zip(slots_h, requests)])
    by_device.step([(s, r[:5]) for s, r in zip(slots_d, requests)])
    for t in range(5, 9):
        tokens = [r[t] for r in requests]
        on_gpu = torch.tensor(tokens, dtype=torch.int32, device="cuda:0")
        a = by_host.step([(s, [tok]) for s, tok in zip(slots_h, tokens)]).clone()
        b = by_device.step([(s, [0]) for s in slots_d], device_tokens=on_gpu).clone()
        assert torch.equal(a, b), f"token {t}"
    check(b[2:3], plain_logits(name, requests[2][:9])[-1:], "bfloat16", "fed from the GPU")
    if graphs:
        assert by_device.graph_replays > 0
    with pytest.raises(StepError, match="device_tokens"):
        by_device.step([(slots_d[0], [1, 2])], device_tokens=on_gpu[:1])          # not a step of single tokens
    with pytest.raises(StepError, match="device_tokens"):
        by_device.step([(s, [0]) for s in slots_d], device_tokens=on_gpu[:2])     # one token short
    assert [by_device.length(s) for s in slots_d] == [9, 9, 9]
    by_host.reset()
    by_device.reset()


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_pass_that_fails_half_way_changes_nothing(dtype, graphs, monkeypatch):
    """A kernel that refuses in the middle of the forward pass (here: the seventh matrix product of
    a step, which lies in the second layer) leaves lengths, block lists and the ledger as they were,
    and the same step, run again, gives the plain implementation's logits: what the failed pass
    wrote lies beyond the committed lengths (src/models/llama/model/decode_tests.rs:762 and
    src/generation/causal_tests.rs:1320 ask the same of the reference)."""
    from burn_transformers_amd.kernels import library as K
    name = "BW"
    engine = engine_for(name, dtype, max_tokens=64 * 5, graphs=graphs)
    first, second = prompts_for(name, [60, 30], seed=77)
    a, b = engine.open(), engine.open()
    engine.step([(a, first[:50]), (b, second[:20])])
    if graphs:                   # decode steps of this shape until they are replayed from a graph
        for t in range(3):
            engine.step([(a, [first[50 + t]]), (b, [second[20 + t]])])
        fed_a, fed_b = 53, 23
    else:
        fed_a, fed_b = 50, 20
    ledger = engine.cache.ledger
    before = (list(ledger.lengths), [list(x) for x in ledger.held_blocks[0]], ledger.blocks[0].available())
    real_gemm, calls = K.gemm, [0]

    def failing(*args, **kwargs):
        calls[0] += 1
        if calls[0] == 7:
            raise K.KernelError("gemm: refused for the test")
        return real_gemm(*args, **kwargs)

    # the step crosses a block's end for sequence a (so a block is reserved) and has a shape that
    # no graph holds yet
    monkeypatch.setattr(K, "gemm", failing)
    with pytest.raises(K.KernelError, match="refused for the test"):
        engine.step([(a, first[fed_a:]), (b, second[fed_b:])])
    assert calls[0] == 7
    monkeypatch.setattr(K, "gemm", real_gemm)
    assert (list(ledger.lengths), [list(x) for x in ledger.held_blocks[0]], ledger.blocks[0].available()) == before
    ledger.check()
    logits = engine.step([(a, first[fed_a:]), (b, second[fed_b:])],
                         want=[list(range(60 - fed_a)), list(range(30 - fed_b))])
    check(logits[:60 - fed_a], plain_logits(name, first)[fed_a:], dtype, "after the failed pass, first")
    check(logits[60 - fed_a:], plain_logits(name, second)[fed_b:], dtype, "after the failed pass, second")
    ledger.check()
    engine.reset()


@pytest.mark.parametrize("name", ["A", "BW"])
def test_greedy_generation_through_the_entry_point(name):
    gain = 6.0
    folder, config, weights = model_folder(name, gain)
    prompts = prompts_for(name, [5, 11, 17], seed=40)
    want = [plain.greedy(p, weights, config, 8) for p in prompts]
    engine = engine_for(name, "float32", gain=gain)
    got = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=8))
    assert [s.token_ids for s in got] == want
    for sequence, prompt in zip(got, prompts):
        assert sequence.prompt_length == len(prompt) and str(sequence.finish_reason) == "Length"
        full = prompt + sequence.token_ids
        ref = torch.log_softmax(plain.forward(full, weights, config), -1)
        for i, (token, logp) in enumerate(zip(sequence.token_ids, sequence.log_probabilities)):
            assert abs(logp - float(ref[len(prompt) - 1 + i, token])) < 1e-4
    chunked = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=8), prefill_chunk=7)
    assert [s.token_ids for s in chunked] == want
    # bfloat16 follows the same path; its tokens may leave the reference where logits nearly tie
    engine16 = engine_for(name, "bfloat16", gain=gain)
    got16 = bt.generate(engine16, prompts, bt.GenerationConfig(max_new_tokens=8))
    same = sum(a == b for s, w in zip(got16, want) for a, b in zip(s.token_ids, w))
    assert same >= 16
    engine.cache.ledger.check()


def test_the_short_way_round_model_random_generate_export():
    """CausalLM.random gives the model that the written folder loads to; model.generate sizes its own
    cache; export_weights gives the stored tensors back."""
    folder, config, weights = model_folder("BW")
    model = bt.CausalLM.random(config, seed=CONFIGS["BW"][1], dtype="float32")
    exported = model.export_weights()
    assert set(exported) == set(weights) and all(torch.equal(exported[k], weights[k]) for k in weights)
    prompts = prompts_for("BW", [4, 30], seed=44)
    got = model.generate(prompts, bt.GenerationConfig(max_new_tokens=6))
    loaded = bt.CausalLM.from_pretrained(folder, dtype="float32")
    same = bt.generate(loaded.engine(max_tokens=256), prompts, bt.GenerationConfig(max_new_tokens=6))
    assert [s.token_ids for s in got] == [s.token_ids for s in same]
    assert [s.token_ids for s in got] == [plain.greedy(p, weights, config, 6) for p in prompts]


def test_unequal_prompts_grown_to_the_position_limit():
    """Prompts of 5, 100 and 127 tokens all decoded to the model's 128 positions in one batch: each
    ends by its own length, the long ones first, and the tokens are the plain greedy loop's."""
    gain = 6.0
    folder, config, weights = model_folder("A", gain)
    limit = config["n_positions"]
    prompts = prompts_for("A", [5, 100, limit - 1], seed=43)
    engine = engine_for("A", "float32", gain=gain, max_tokens=3 * 128)
    with pytest.raises(bt.GenerationError, match="need 204 positions, the limit is 128"):
        bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=200))
    order = []
    got = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=200), total_length=limit,
                      on_token=lambda row, token, logp, reason: order.append(row) if reason is not None else None)
    assert [len(s.token_ids) for s in got] == [limit - 5, limit - 100, 1]
    assert all(str(s.finish_reason) == "Length" for s in got)
    assert order == [2, 1, 0]
    for prompt, sequence in zip(prompts, got):
        assert sequence.token_ids == plain.greedy(prompt, weights, config, len(sequence.token_ids))
    engine.cache.ledger.check()


def test_sampling_end_of_sequence_and_batches():
    folder, config, weights = model_folder("BW", 6.0)
    engine = engine_for("BW", "float32", gain=6.0, max_tokens=64 * 3)
    prompts = prompts_for("BW", [1, 23, 9, 30, 2], seed=41)
    cfg = bt.GenerationConfig(max_new_tokens=12, strategy="sample", temperature=0.8, seed=7)
    first = bt.generate(engine, prompts, cfg, prefill_chunk=7, batch_size=2)
    again = bt.generate(engine, prompts, cfg, batch_size=2)
    assert [s.token_ids for s in first] == [s.token_ids for s in again]
    other = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=12, strategy="sample",
                                                             temperature=0.8, seed=8), batch_size=2)
    assert [s.token_ids for s in first] != [s.token_ids for s in other]
    # every sampled token is the inverse-CDF choice of the plain implementation for its draw
    for batch_start in (0, 2, 4):
        rows = list(range(batch_start, min(batch_start + 2, len(prompts))))
        for b, index in enumerate(rows):
            full = prompts[index] + first[index].token_ids
            logits = plain.forward(full, weights, config)
            for s, token in enumerate(first[index].token_ids):
                u = plain.interior_unit(plain.splitmix64(7, s * len(rows) + b))
                z = logits[len(prompts[index]) - 1 + s]
                p = torch.cumsum(torch.softmax(z / 0.8, -1), -1)
                lo = float(p[token - 1]) if token else 0.0
                assert lo - 1e-4 <= u <= float(p[token]) + 1e-4
    # an end-of-sequence token ends its row, the others go on
    greedy = bt.generate(engine, prompts[:3], bt.GenerationConfig(max_new_tokens=10))
    eos = greedy[1].token_ids[3]
    stopped = bt.generate(engine, prompts[:3], bt.GenerationConfig(max_new_tokens=10, eos_token_ids=[eos]))
    cut = greedy[1].token_ids.index(eos) + 1
    assert stopped[1].token_ids == greedy[1].token_ids[:cut]
    assert str(stopped[1].finish_reason) == f"EndOfSequence(token_id={eos})"
    for i in (0, 2):
        if eos not in greedy[i].token_ids:
            assert stopped[i].token_ids == greedy[i].token_ids
    engine.cache.ledger.check()
    assert engine.cache.ledger.slots.available() == engine.cache.max_slots


@pytest.mark.parametrize("dtype", DTYPES)
def test_tiny_b_prompts_of_1_and_23_in_chunks_of_7_then_12_sampled_tokens(dtype):
    """The second tiny configuration exactly as it is stated (3 layers, width 96, 2 heads of 48,
    inner width 320, 517 tokens, 64 positions, exact GELU, eps 1e-6, scores divided by layer + 1):
    prompts of 1 and 23 tokens fed in chunks of 7 (the first request is idle in chunks two to
    four), then 12 tokens sampled at temperature 0.8 from a fixed seed.  Every sampled token is the
    plain implementation's inverse-CDF choice for its draw, the log-probabilities are its
    log-softmax, and feeding the prompts whole gives the same tokens."""
    folder, config, weights = model_folder("B", 6.0)
    assert config["n_positions"] == 64
    engine = engine_for("B", dtype, gain=6.0, max_tokens=128)
    prompts = prompts_for("B", [1, 23], seed=45)
    cfg = bt.GenerationConfig(max_new_tokens=12, strategy="sample", temperature=0.8, seed=11)
    chunked = bt.generate(engine, prompts, cfg, prefill_chunk=7)
    whole = bt.generate(engine, prompts, cfg)
    band = 1e-4 if dtype == "float32" else 3e-2
    if dtype == "float32":
        assert [s.token_ids for s in chunked] == [s.token_ids for s in whole]
    for b, (prompt, sequence) in enumerate(zip(prompts, chunked)):
        assert len(sequence.token_ids) == 12 and str(sequence.finish_reason) == "Length"
        logits = plain.forward(prompt + sequence.token_ids, weights, config)
        for s, (token, logp) in enumerate(zip(sequence.token_ids, sequence.log_probabilities)):
            u = plain.interior_unit(plain.splitmix64(11, s * 2 + b))
            z = logits[len(prompt) - 1 + s]
            c = torch.cumsum(torch.softmax(z / 0.8, -1), -1)
            low = float(c[token - 1]) if token else 0.0
            assert low - band <= u <= float(c[token]) + band, f"row {b} step {s}"
            assert abs(logp - plain.log_probability(z, token, 0.8)) < (1e-4 if dtype == "float32" else 6e-2)
    engine.cache.ledger.check()


def test_command_line(capsys, tmp_path):
    """gpt2_generate MODEL_DIR PROMPT MAX_NEW_TOKENS, the reference's positional arguments
    (examples/llama_generate.rs:66-81)."""
    import json
    from burn_transformers_amd.cli import main
    folder, config, weights = model_folder("A", 6.0)
    prompts = prompts_for("A", [6, 13], seed=60)
    text = ";".join(",".join(str(t) for t in p) for p in prompts)
    assert main([folder, text, "5", "--dtype", "float32", "--json", "--load-report"]) == 0
    captured = capsys.readouterr()
    lines = [json.loads(line) for line in captured.out.strip().splitlines()]
    report = json.loads([line for line in captured.err.splitlines() if line.startswith("{")][-1])
    assert report["applied"] == len(weights) and report["namespace"] == "" and report["ignored"] == []
    assert [line["token_ids"] for line in lines] == [plain.greedy(p, weights, config, 5) for p in prompts]
    assert all(line["finish_reason"] == "Length" for line in lines)
    assert main([folder, text, "0"]) == 2 and main([folder, text, "3", "4"]) == 2
    with pytest.raises(SystemExit, match="tokenizer.json"):
        main([folder])                                  # the default prompt is text
    # random-weights mode writes the folder first
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(config))
    assert main([str(tmp_path / "made"), "1,2,3", "4", "--random-weights", str(cfg_path), "--weights-seed", "3",
                 "--temperature", "0.7", "--seed", "5"]) == 0
    assert sorted(p.name for p in (tmp_path / "made").iterdir()) == ["config.json", "model.safetensors"]
