"""Launch lists: a step's kernel calls kept as (entry point, structure) pairs and walked in C++.

A list is recorded from the same parts that issue kernels one by one, so both ways run the same
kernels with the same arguments: every result here is compared bit for bit."""

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from model_helpers import model_folder, plain_logits, prompts_for, tolerance  # noqa: E402

_models = {}


def model_for(name, dtype):
    if (name, dtype) not in _models:
        folder, _, _ = model_folder(name)
        _models[(name, dtype)] = bt.load_model(folder, dtype=dtype, device="cuda:0")
    return _models[(name, dtype)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "BW", "C"])
def test_steps_from_launch_lists_equal_steps_issued_one_by_one(name, dtype):
    """A random schedule of prompts, chunks and single tokens on two engines of one model, one
    walking launch lists and one calling every kernel from Python; no graphs in either."""
    model = model_for(name, dtype)
    assert model.recordable
    listed = bt.Engine(model, max_tokens=64 * 12, graphs=False)
    direct = bt.Engine(model, max_tokens=64 * 12, graphs=False, programs=False)
    assert listed.use_programs and not direct.use_programs
    gen = torch.Generator().manual_seed(3)
    limit = model.max_positions
    requests = prompts_for(name, [limit - 3, 40, 70, 9], seed=81)
    slots = [(listed.open(), direct.open()) for _ in requests]
    fed = [0] * len(requests)
    shapes = set()
    for turn in range(40):
        live = [i for i in range(len(requests)) if fed[i] < len(requests[i])]
        if not live:
            break
        chosen = [i for i in live if int(torch.randint(0, 3, (1,), generator=gen)) > 0] or live[:1]
        counts = [1 if turn % 3 == 2 else int(torch.randint(1, 24, (1,), generator=gen)) for _ in chosen]
        entries_l = [(slots[i][0], requests[i][fed[i]:fed[i] + c]) for i, c in zip(chosen, counts)]
        entries_d = [(slots[i][1], requests[i][fed[i]:fed[i] + c]) for i, c in zip(chosen, counts)]
        want = [list(range(len(e[1]))) for e in entries_l]
        a = listed.step(entries_l, want).clone()
        b = direct.step(entries_d, want).clone()
        assert torch.equal(a, b), f"turn {turn}"
        shapes.add(tuple(len(e[1]) for e in entries_l))
        for i, e in zip(chosen, entries_l):
            fed[i] += len(e[1])
    # a shape's first step launches as it records; every later one runs from its list (the lists kept
    # now may be none: a workspace that grows in the last step drops them all)
    assert 0 < listed.program_runs < listed.steps_run and direct.program_runs == 0
    # and against the plain implementation, through the list that was used most recently
    ids = requests[1]
    slot = listed.open()
    logits = listed.step([(slot, ids)], want=[list(range(len(ids)))])
    want = plain_logits(name, ids)
    assert float((logits.cpu().double() - want).abs().max()) <= tolerance(dtype, want)
    listed.reset()
    direct.reset()


def test_a_repeated_shape_reuses_its_list_and_a_grown_workspace_makes_lists_stale():
    model = model_for("A", "bfloat16")
    engine = bt.Engine(model, max_tokens=64 * 40, graphs=False)
    ids = prompts_for("A", [20], seed=82)[0]
    want = plain_logits("A", ids)
    outs = []
    for _ in range(3):
        slot = engine.open()
        outs.append(engine.step([(slot, ids)], want=[list(range(20))]).clone())
        engine.close(slot)
    assert len(engine._programs) == 1 and engine.program_runs == 2
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    # a much larger step makes the workspaces grow: the old list names addresses that are gone
    many = prompts_for("A", [120] * 16, seed=83)
    slots = [engine.open() for _ in many]
    engine.step(list(zip(slots, many)))
    for slot in slots:
        engine.close(slot)
    slot = engine.open()
    again = engine.step([(slot, ids)], want=[list(range(20))]).clone()
    assert torch.equal(again, outs[0])
    assert float((again.cpu().double() - want).abs().max()) <= tolerance("bfloat16", want)


def test_a_call_that_refuses_names_itself_and_the_step_changes_nothing():
    """The walk stops at the call that refuses; the message is that kernel's own."""
    model = model_for("A", "float32")
    engine = bt.Engine(model, max_tokens=256, graphs=False)
    slot = engine.open()
    ids = prompts_for("A", [30], seed=84)[0]
    engine.step([(slot, ids[:10])])
    program = engine.last_program
    # break one call of the recorded list: a product of rows that no kernel takes
    index = next(i for i, (_, name, _) in enumerate(program.calls) if name == "bt_gemm_skinny_call")
    call = program.calls[index][2]
    rows = call.M
    call.M = 65
    slot2 = engine.open()
    before = (engine.length(slot2), list(engine.cache.blocks(slot2)))
    with pytest.raises(K.KernelError, match=r"gemm_skinny: 65 rows, at most 64 \(call \d+ of \d+, bt_gemm_skinny_call\)"):
        engine.step([(slot2, ids[:10])])
    assert (engine.length(slot2), list(engine.cache.blocks(slot2))) == before
    engine.cache.ledger.check()
    call.M = rows
    logits = engine.step([(slot2, ids[:10])])
    want = plain_logits("A", ids[:10])[-1:]
    assert float((logits.cpu().double() - want).abs().max()) <= tolerance("float32", want)


@pytest.mark.parametrize("gpu_is_the_limit", [False, True])
def test_a_measured_shape_is_captured_or_left_to_its_list(gpu_is_the_limit, monkeypatch):
    """The engine's own choice (graphs=True) with the verdict of the measurement given: a repeating
    shape runs from Python once (its list is recorded), from its list while it is measured, and
    then from a graph if the host was found to be the limit, else from its list for good.  The
    logits are the plain implementation's on either path."""
    from burn_transformers_amd.engine import engine as engine_module
    seen = []

    def verdict(samples):
        seen.append(samples)
        return gpu_is_the_limit

    monkeypatch.setattr(engine_module, "launch_bound", verdict)
    model = model_for("A", "bfloat16")
    engine = bt.Engine(model, max_tokens=256)
    assert engine.use_graphs and engine.use_programs
    ids = prompts_for("A", [40], seed=86)[0]
    slot = engine.open()
    rows = [engine.step([(slot, ids[:8])], want=[list(range(8))]).clone()]
    for t in range(8, 40):
        rows.append(engine.step([(slot, [ids[t]])]).clone())
    probes = engine_module._PROBES
    assert len(seen) == 1 and len(seen[0]) == probes and all(gpu > 0 and host > 0 for gpu, host in seen[0])
    if gpu_is_the_limit:
        assert engine.graphs_declined == 1 and engine.graph_replays == 0 and engine.program_runs == 32 - 1
    else:
        # the first step records, the next are measured from the list, the rest are replayed
        assert engine.graphs_declined == 0 and engine.graph_replays == 32 - 1 - probes and engine.program_runs == probes
    want = plain_logits("A", ids)
    assert float((torch.cat(rows).cpu().double() - want).abs().max()) <= tolerance("bfloat16", want)


def test_the_engine_chooses_a_path_for_a_repeating_shape_by_itself():
    """The same without a given verdict: whatever this machine's clocks say, the decision is taken
    once, the steps run from the list or from a graph, and the logits are right."""
    model = model_for("A", "bfloat16")
    engine = bt.Engine(model, max_tokens=256)
    ids = prompts_for("A", [40], seed=87)[0]
    slot = engine.open()
    rows = [engine.step([(slot, ids[:8])], want=[list(range(8))]).clone()]
    for t in range(8, 40):
        rows.append(engine.step([(slot, [ids[t]])]).clone())
    decisions = [v for v in engine._launch_bound.values() if isinstance(v, bool)]
    assert len(decisions) == 1
    assert engine.graph_replays + engine.program_runs == 32 - 1
    assert (engine.graph_replays > 0) == (decisions[0] is False)
    want = plain_logits("A", ids)
    assert float((torch.cat(rows).cpu().double() - want).abs().max()) <= tolerance("bfloat16", want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "BW"])
def test_one_launch_list_serves_every_prompt_length_of_its_class(name, dtype):
    """Prompts of 65 to 128 tokens (and 129 to 190), in random order, on an engine that walks launch
    lists and on one that issues every kernel from Python: the same bits, and the first engine has
    recorded ONE list for each class of lengths (65 .. 128, 129 .. 192), whose counts it sets to
    each step's; a step with other wanted rows, or of several sequences, is another class."""
    model = model_for(name, dtype)
    listed = bt.Engine(model, max_tokens=64 * 8, graphs=False)
    direct = bt.Engine(model, max_tokens=64 * 8, graphs=False, programs=False)
    gen = torch.Generator().manual_seed(17)
    limit = model.max_positions
    lengths = [65, 128, 70, 127, 100, 66, 96] + torch.randint(65, 129, (8,), generator=gen).tolist()
    if limit >= 190:
        lengths += [129, 190, 150, 64, 65]
    lengths = [n for n in lengths if n < limit]            # (one more token follows every prompt)
    classes = {n if n <= 64 else (n + 63) // 64 for n in lengths}

    def walk(order):
        for n in order:
            ids = prompts_for(name, [n], seed=1000 + n)[0]
            a, b = listed.open(), direct.open()
            got, want = listed.step([(a, ids)]).clone(), direct.step([(b, ids)])
            assert torch.equal(got, want), f"a prompt of {n} tokens"
            # the cache holds the same too: one more token on both gives the same bits
            got, want = listed.step([(a, [ids[0]])]).clone(), direct.step([(b, [ids[0]])])
            assert torch.equal(got, want), f"the token after a prompt of {n} tokens"
            listed.close(a)
            direct.close(b)
        return ids

    # One prompt of every class, the longest first, twice over: the workspaces then have their sizes
    # (a list recorded while one grew is not kept, and growth drops the older lists) and every class
    # has its list.  From then on no step of any of these lengths is issued from Python again.
    firsts = sorted({max(n for n in lengths if (n if n <= 64 else (n + 63) // 64) == c) for c in classes}, reverse=True)
    walk(firsts + firsts)
    recorded, runs, steps = listed.programs_recorded, listed.program_runs, listed.steps_run
    ids = walk(lengths)
    assert listed.programs_recorded == recorded, f"{listed.programs_recorded - recorded} steps were issued from Python again"
    assert listed.program_runs - runs == listed.steps_run - steps == 2 * len(lengths)
    assert len(listed._programs) == len(classes) + 1           # one list a class, and the step of one token
    assert direct.program_runs == 0
    # the last prompt against the plain implementation: the lists are not only equal to the direct path
    reference = plain_logits(name, ids)[-1:]
    logits = listed.step([(listed.open(), ids)])
    assert float((logits.cpu().double() - reference).abs().max()) <= tolerance(dtype, reference)
    # two sequences of unequal lengths, all rows wanted for one of them: classes of their own
    first, second = prompts_for(name, [70, 30], seed=5)
    for _ in range(2):
        a, b = (listed.open(), listed.open()), (direct.open(), direct.open())
        for cut in ((40, 30), (30, 0)):
            entries = [(first[:40] if cut[0] == 40 else first[40:]), (second if cut[1] else [])]
            want_rows = [list(range(len(entries[0]))), []]
            got = listed.step(list(zip(a, entries)), want=want_rows).clone()
            want = direct.step(list(zip(b, entries)), want=want_rows)
            assert torch.equal(got, want)
        for slot in a:
            listed.close(slot)
        for slot in b:
            direct.close(slot)
    listed.reset()
    direct.reset()
    listed.cache.ledger.check()
