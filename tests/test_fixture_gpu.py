"""The engine against the reference's own vector, and at head sizes that no MFMA kernel takes.

src/models/gpt2/fixtures/tiny_reference.json holds PyTorch's logits for a GPT-2 of width 12 with
3 heads (head size 4), inner width 17, 19 tokens and 16 positions, whose weights come from the
xorshift generator of src/models/gpt2/prepare_reference.py:19-38; the reference compares itself
with it in src/models/gpt2/model_tests.rs:154-206.  Here the ENGINE's float32 logits are compared
with that vector directly, not through the plain implementation of the tests.  A head size of 4
runs on the plain product and the plain attention kernel; bfloat16 has no kernels for it and says
so when the model is built."""

import json

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from model_helpers import tolerance  # noqa: E402
from test_plain import FIXTURE, fixture_weights  # noqa: E402


def fixture():
    with open(FIXTURE) as handle:
        return json.load(handle)


@pytest.mark.parametrize("activation", ["gelu_new", "gelu"])
def test_engine_gives_the_reference_vector(activation):
    reference = fixture()
    weights = fixture_weights(reference["parameter_shapes"])
    config = dict(reference["config"], activation_function=activation)
    model = bt.model_from_tensors(config, weights, dtype="float32", device="cuda:0")
    assert model.blocks[0].mixers()[0].head_dim == 4
    expected = reference["references"][activation]["logits"]
    requests = [ids[:sum(mask)] for ids, mask in zip(reference["input_ids"], reference["token_mask"])]
    want = [torch.tensor(expected[row])[:len(ids)] for row, ids in enumerate(requests)]
    engine = bt.Engine(model, max_tokens=256)
    # both requests whole, as one ragged batch (4 and 3 tokens)
    slots = [engine.open() for _ in requests]
    logits = engine.step(list(zip(slots, requests)), want=[list(range(len(r))) for r in requests]).cpu()
    assert (logits[:4] - want[0]).abs().max() <= 2e-5 and (logits[4:] - want[1]).abs().max() <= 2e-5
    for slot in slots:
        engine.close(slot)
    # token by token, the two requests side by side until the shorter one has ended
    slots = [engine.open() for _ in requests]
    rows = [[], []]
    for t in range(4):
        live = [i for i, r in enumerate(requests) if t < len(r)]
        logits = engine.step([(slots[i], [requests[i][t]]) for i in live]).cpu()
        for row, i in enumerate(live):
            rows[i].append(logits[row])
    for i in range(2):
        assert (torch.stack(rows[i]) - want[i]).abs().max() <= 2e-5, f"request {i} token by token"
    # a prompt, then the rest one by one; the slot was used before
    engine.close(slots[0])
    slot = engine.open()
    head = engine.step([(slot, requests[0][:2])], want=[[0, 1]]).cpu().clone()
    tail = [engine.step([(slot, [t])]).cpu().clone() for t in requests[0][2:]]
    assert (torch.cat([head] + tail) - want[0]).abs().max() <= 2e-5
    engine.cache.ledger.check()


def test_bfloat16_says_which_head_sizes_it_takes():
    reference = fixture()
    weights = fixture_weights(reference["parameter_shapes"])
    with pytest.raises(ValueError, match=r"bfloat16 kernels take head sizes 16, 32, ... 128, not 4.*float32"):
        bt.model_from_tensors(reference["config"], weights, dtype="bfloat16", device="cuda:0")


# a width that four does not divide (so every product is the plain one), heads of five channels
ODD = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 15, "n_head": 3,
       "n_inner": 22, "vocab_size": 61, "n_positions": 140, "activation_function": "gelu_new",
       "layer_norm_epsilon": 1e-4, "scale_attn_by_inverse_layer_idx": True}
# heads of 24 and of 136: multiples of four and of eight that are no multiple of 16, or beyond 128
HEADS = [dict(ODD, n_embd=48, n_head=2, n_inner=64), dict(ODD, n_embd=136, n_head=1, n_inner=40)]


@pytest.mark.parametrize("config", [ODD] + HEADS, ids=["head5", "head24", "head136"])
def test_any_head_size_in_float32(config):
    """Whole, in chunks and token by token across a block's end, in a ragged batch, against the plain
    implementation."""
    _, tensors = bt.random_tensors(config, 5)
    tensors = {k: (v * 4.0 if v.dim() == 2 else v) for k, v in tensors.items()}
    model = bt.model_from_tensors(config, tensors, dtype="float32", device="cuda:0")
    engine = bt.Engine(model, max_tokens=512)
    gen = torch.Generator().manual_seed(6)
    requests = [torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist() for n in (130, 7, 66)]
    want = [plain.forward(r, tensors, config) for r in requests]
    slots = [engine.open() for _ in requests]
    got = [[] for _ in requests]
    heads = [60, 3, 66]
    logits = engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, heads)],
                         want=[list(range(n)) for n in heads]).cpu().clone()
    at = 0
    for i, n in enumerate(heads):
        got[i].append(logits[at:at + n])
        at += n
    engine.close(slots[2])
    position = list(heads)
    for chunk in (1, 1, 1, 1, 5, 1, 64, 1):        # request 1 ends after four tokens, request 0 crosses 64 and 128
        live = [i for i in (0, 1) if position[i] < len(requests[i])]
        if not live:
            break
        entries = [(slots[i], requests[i][position[i]:position[i] + chunk]) for i in live]
        logits = engine.step(entries, want=[list(range(len(e[1]))) for e in entries]).cpu().clone()
        at = 0
        for i, e in zip(live, entries):
            got[i].append(logits[at:at + len(e[1])])
            at += len(e[1])
            position[i] += len(e[1])
    for i, r in enumerate(requests):
        rows = torch.cat(got[i]).double()
        assert rows.shape[0] == len(r), (i, rows.shape)
        err = float((rows - want[i]).abs().max())
        assert err <= tolerance("float32", want[i]), f"request {i}: {err}"
    engine.reset()
    engine.cache.ledger.check()
