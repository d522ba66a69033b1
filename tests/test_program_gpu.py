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
    # a shape's first step launches as it records; every later one runs from its list
    assert listed.program_runs < listed.steps_run and len(listed._programs) > 0 and direct.program_runs == 0
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
