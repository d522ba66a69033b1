"""Float32 matrices that bfloat16 cannot hold, through loader, packed copies and every kind of step.

The other engine tests store their random weights in bfloat16, so a float32 engine that rounded its
matrices through bfloat16 somewhere (in the loader, in a packed second copy, in a chunk-major
buffer) would pass them.  Here the checkpoint holds full 24-bit values, and the test first shows
that rounding them would be seen: the plain implementation on rounded weights differs from the plain
implementation on the stored ones by many times the bound that the engine is held to."""

import tempfile

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from model_helpers import CONFIGS, prompts_for, tolerance  # noqa: E402

_held = {}


def full_precision_model(name):
    """(folder, config, the float32 weights as stored) with matrices scaled up so that the logits
    are not nearly uniform; written once per process."""
    if name not in _held:
        config, seed = CONFIGS[name]
        holder = tempfile.TemporaryDirectory(prefix=f"bt_full_{name}_")
        weights = bt.write_random_model(holder.name, config, seed, store_dtype="float32")
        weights = {k: (v * 4.0 if v.dim() == 2 else v) for k, v in weights.items()}
        bt.write_safetensors(f"{holder.name}/model.safetensors", weights)
        assert any((v.to(torch.bfloat16).float() != v).any() for v in weights.values())
        _held[name] = (holder, config, weights)
    holder, config, weights = _held[name]
    return holder.name, config, weights


def check(got, want, dtype, what):
    error = float((got.detach().cpu().double() - want).abs().max())
    assert error <= tolerance(dtype, want), f"{what}: max abs error {error} > {tolerance(dtype, want)}"


@pytest.mark.parametrize("name", ["A", "BW"])
def test_float32_weights_keep_all_their_bits(name):
    folder, config, weights = full_precision_model(name)
    rounded = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    limit = config["n_positions"]
    ids = prompts_for(name, [min(100, limit - 2)], seed=5)[0]
    want = plain.forward(ids, weights, config)
    seen_if_rounded = float((plain.forward(ids, rounded, config) - want).abs().max())
    assert seen_if_rounded > 20 * tolerance("float32", want), "rounding the weights would not show in this test"

    model = bt.load_model(folder, dtype="float32", device="cuda:0")
    assert model.load_report["converted"] == {}, model.load_report          # nothing changed precision
    for name_, tensor in model.export_weights().items():
        assert torch.equal(tensor, weights[name_]), name_
    engine = bt.Engine(model, max_tokens=64 * 40, graphs=False)
    # whole
    slot = engine.open()
    check(engine.step([(slot, ids)], want=[list(range(len(ids)))]), want, "float32", f"{name} whole")
    engine.close(slot)
    # the last 32 tokens one by one (products read the packed second copies of the matrices)
    slot = engine.open()
    cut = len(ids) - 32
    rows = [engine.step([(slot, ids[:cut])], want=[list(range(cut))]).clone()]
    for t in range(cut, len(ids)):
        rows.append(engine.step([(slot, [ids[t]])]).clone())
    check(torch.cat(rows), want, "float32", f"{name} tail one by one")
    engine.close(slot)
    # decode batches of 8 rows (packed copies, row-major rows) and of 17 rows (chunk-major rows)
    for batch in (8, 17):
        lengths = [3 + (5 * i) % 40 for i in range(batch)]
        requests = prompts_for(name, [n + 4 for n in lengths], seed=batch)
        slots = [engine.open() for _ in requests]
        engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, lengths)], want=[[] for _ in requests])
        got = [[] for _ in requests]
        for t in range(4):
            logits = engine.step([(s, [r[n + t]]) for s, r, n in zip(slots, requests, lengths)]).clone()
            for i in range(batch):
                got[i].append(logits[i:i + 1])
        for i, (r, n) in enumerate(zip(requests, lengths)):
            check(torch.cat(got[i]), plain.forward(r, weights, config)[n:], "float32", f"{name} batch {batch} row {i}")
        for s in slots:
            engine.close(s)
    engine.cache.ledger.check()


@pytest.mark.parametrize("name", ["A", "BW"])
def test_a_float32_checkpoint_run_in_bfloat16_is_rounded_once(name):
    """``dtype=bfloat16`` of a checkpoint stored in 32-bit: matrices are rounded to nearest even,
    once, and vectors stay in float32 (src/checkpoint/runtime/convert.rs:10-20)."""
    folder, config, weights = full_precision_model(name)
    model = bt.load_model(folder, dtype="bfloat16", device="cuda:0")
    assert set(model.load_report["converted"]) == {"float32->bfloat16"}
    rounded = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in weights.items()}
    for name_, tensor in model.export_weights().items():
        assert torch.equal(tensor, rounded[name_]), name_
    ids = prompts_for(name, [70], seed=6)[0]
    engine = bt.Engine(model, max_tokens=256, graphs=False)
    slot = engine.open()
    check(engine.step([(slot, ids)], want=[list(range(len(ids)))]), plain.forward(ids, rounded, config), "bfloat16",
          f"{name} bfloat16 from a float32 checkpoint")
    engine.close(slot)
