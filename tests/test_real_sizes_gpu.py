"""The engine at the sizes of real models: two layers of GPT-2 XL's width, and all twelve layers
of GPT-2 small's (at the end of the file).

The engine at the layer sizes of GPT-2 XL (width 1600, 25 heads of 64, inner 6400, vocabulary
50257, 1,024 positions) with two layers, against the plain implementation in float64: the sizes
the measured kernels run at (columns per work-group chosen by balance, split K, paired and
LDS-shared prefill attention, hundreds of keys per query) are not the tiny configurations'.

Random weights of the initialiser give nearly uniform attention, under which a lost block of
keys barely moves a bfloat16 logit; the query and key thirds of the fused projection are scaled
up so that each query has a few dominant keys somewhere among its hundreds."""

import os
import tempfile

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from model_helpers import tolerance  # noqa: E402

WIDE = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 1600, "n_head": 25,
        "n_inner": 6400, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
        "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
SHARPEN = 2.5        # on queries and on keys: scores 6.25 times those of the initialiser
DTYPES = ["float32", "bfloat16"]
_state = {}


def wide_model():
    """(folder, weights as stored, rounded to bfloat16 and widened again); made once per process."""
    if not _state:
        holder = tempfile.TemporaryDirectory(prefix="bt_wide_")
        weights = bt.write_random_model(holder.name, WIDE, 3)
        d = WIDE["n_embd"]
        for layer in range(WIDE["n_layer"]):
            weights[f"h.{layer}.attn.c_attn.weight"][:, :2 * d] *= SHARPEN       # Conv1D layout [in, out]
            weights[f"h.{layer}.attn.c_attn.bias"][:2 * d] *= SHARPEN
        stored = {k: (v.to(torch.bfloat16) if v.dim() == 2 else v) for k, v in weights.items()}
        bt.write_safetensors(os.path.join(holder.name, "model.safetensors"), stored)
        _state.update(holder=holder, weights={k: v.float() for k, v in stored.items()}, models={})
    return _state["holder"].name, _state["weights"]


def engine_for(dtype, max_tokens=4096):
    folder, _ = wide_model()
    if dtype not in _state["models"]:
        _state["models"][dtype] = bt.load_model(folder, dtype=dtype, device="cuda:0")
    return bt.Engine(_state["models"][dtype], max_tokens=max_tokens)


def request(length, seed):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, WIDE["vocab_size"], (length,), generator=gen).tolist()


def plain_rows(ids, rows):
    """float64 logits of the plain implementation at ``rows`` of the request."""
    _, weights = wide_model()
    return plain.forward(ids, weights, WIDE, rows=rows)


# bfloat16 under sharpened attention: a score of magnitude 15 computed from queries and keys rounded
# to 8 bits is off by about 15 * 2^-8 = 0.06, so a weight of the softmax by 6 %, where the
# initialiser's nearly uniform attention would hide both this and a lost key.  Measured over this
# file's cases: 1.2e-2 to 1.6e-2 of the largest logit.  What a tolerance of this size could hide
# is covered by the tests of the attention kernels in which one key takes all the weight.
BF16_BOUND = 2.5e-2


def check(got, want, dtype, what):
    got = got.detach().cpu().double()
    err = float((got - want).abs().max())
    assert torch.isfinite(got).all(), what
    bound = tolerance(dtype, want) if dtype == "float32" else BF16_BOUND * float(want.abs().max())
    print(f"[real sizes] {what} ({dtype}): max abs error {err:.3g}, {err / float(want.abs().max()):.3g} of the largest logit", flush=True)
    assert err <= bound, f"{what}: max abs error {err} > {bound}"


def test_attention_of_the_wide_model_is_peaked():
    """The premise of this file: among hundreds of keys a query's largest weight is far above uniform."""
    _, weights = wide_model()
    ids = request(600, seed=1)
    w = {k: v.double() for k, v in weights.items()}
    x = w["wte.weight"][ids] + w["wpe.weight"][:len(ids)]
    h = plain.layer_norm(x, w["h.0.ln_1.weight"], w["h.0.ln_1.bias"], 1e-5)
    qkv = h @ w["h.0.attn.c_attn.weight"] + w["h.0.attn.c_attn.bias"]
    d = WIDE["n_embd"]
    q, k = plain.split_heads(qkv[:, :d], 25), plain.split_heads(qkv[:, d:2 * d], 25)
    scores = (q[:, -1:] @ k.transpose(-1, -2)) * 64 ** -0.5                   # the last query of every head
    top = torch.softmax(scores, -1).max(-1).values
    assert float(top.median()) > 20.0 / len(ids)


@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_request(dtype):
    engine = engine_for(dtype)
    ids = request(700, seed=2)
    rows = list(range(0, 700, 41)) + [63, 64, 127, 128, 698, 699]
    slot = engine.open()
    logits = engine.step([(slot, ids)], want=[rows])
    check(logits, plain_rows(ids, rows), dtype, "whole request of 700")
    engine.close(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prompts_in_chunks_that_start_off_the_block_grid(dtype):
    """Two requests fed in chunks of 200 and 130 tokens: chunks start at 200, 400, 600 and at 130,
    260, ..., none a multiple of the cache's blocks of 64 or the kernels' tiles of 128 queries."""
    engine = engine_for(dtype)
    requests = [request(700, seed=2), request(520, seed=5)]
    chunks, fed, slots = [200, 130], [0, 0], [engine.open(), engine.open()]
    got, rows = [[], []], [[], []]
    while any(f < len(r) for f, r in zip(fed, requests)):
        live = [i for i in range(2) if fed[i] < len(requests[i])]
        entries = [(slots[i], requests[i][fed[i]:fed[i] + chunks[i]]) for i in live]
        wants = [[0, len(e[1]) // 2, len(e[1]) - 1] for e in entries]
        logits = engine.step(entries, want=wants).clone()
        for n, i in enumerate(live):
            got[i].append(logits[3 * n:3 * n + 3])
            rows[i] += [fed[i] + w for w in wants[n]]
            fed[i] += len(entries[n][1])
    for i, r in enumerate(requests):
        check(torch.cat(got[i]), plain_rows(r, rows[i]), dtype, f"request {i} in chunks of {chunks[i]}")
    for slot in slots:
        engine.close(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_last_32_tokens_one_by_one_up_to_the_position_limit(dtype):
    engine = engine_for(dtype)
    ids = request(1024, seed=3)
    slot = engine.open()
    head = len(ids) - 32
    got = [engine.step([(slot, ids[:head])], want=[[0, 500, head - 1]]).clone()]
    for t in range(head, len(ids)):
        got.append(engine.step([(slot, [ids[t]])]).clone())
    check(torch.cat(got), plain_rows(ids, [0, 500, head - 1] + list(range(head, len(ids)))), dtype, "tail of 1,024")
    assert engine.graph_replays + engine.program_runs > 0
    engine.close(slot)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_batches_one_after_another(dtype):
    """Prompts of unequal length in one step, then one token each; shorter requests end earlier and
    the next batch takes their slots."""
    engine = engine_for(dtype, max_tokens=2048)
    seen = []
    for b, (lengths, extra) in enumerate([([900, 300, 65], [6, 3, 9]), ([130, 700, 1, 64], [4, 8, 12, 2])]):
        requests = [request(n + e, seed=20 + 10 * b + i) for i, (n, e) in enumerate(zip(lengths, extra))]
        slots = [engine.open() for _ in requests]
        seen.append(list(slots))
        wants = [[0, n // 2, n - 1] if n > 1 else [0] for n in lengths]
        rows = [list(w) for w in wants]
        logits = engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, lengths)], want=wants).clone()
        got, at = [], 0
        for w in wants:
            got.append([logits[at:at + len(w)]])
            at += len(w)
        live, position = list(range(len(requests))), list(lengths)
        while live:
            logits = engine.step([(slots[i], [requests[i][position[i]]]) for i in live]).clone()
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                rows[i].append(position[i])
                position[i] += 1
            for i in [i for i in live if position[i] >= len(requests[i])]:
                engine.close(slots[i])
                live.remove(i)
        for i, r in enumerate(requests):
            check(torch.cat(got[i]), plain_rows(r, rows[i]), dtype, f"batch {b} request {i}")
        engine.cache.ledger.check()
    assert set(seen[0]) & set(seen[1]), "slots were not used again"


# --- GPT-2 small's sizes with all twelve layers, in float32 and in bfloat16: depth ----------------

LONG = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 256, "n_head": 4,
        "n_inner": 512, "vocab_size": 1000, "n_positions": 4096, "activation_function": "gelu_new",
        "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}


@pytest.mark.parametrize("dtype", DTYPES)
def test_chunks_of_a_prompt_behind_a_long_context(dtype):
    """A request of 3,300 tokens fed in chunks of 256 (heads of 64, room for 4,096 positions, attention
    sharpened): from 1,024 tokens of context on the bfloat16 attention kernel cuts the keys of its two query
    tiles into runs that separate work-groups take and a second kernel joins.  The logits at the
    first, a middle and the last place of every chunk against the plain implementation, and a
    second request beside it whose chunks are shorter than a tile."""
    from types import SimpleNamespace
    with tempfile.TemporaryDirectory(prefix="bt_long_") as folder:
        weights = bt.write_random_model(folder, LONG, 12)
        d = LONG["n_embd"]
        for layer in range(LONG["n_layer"]):
            weights[f"h.{layer}.attn.c_attn.weight"][:, :2 * d] *= 4.0
            weights[f"h.{layer}.attn.c_attn.bias"][:2 * d] *= 4.0
        stored = {k: (v.to(torch.bfloat16) if v.dim() == 2 else v) for k, v in weights.items()}
        bt.write_safetensors(os.path.join(folder, "model.safetensors"), stored)
        weights = {k: v.float() for k, v in stored.items()}
        model = bt.load_model(folder, dtype=dtype, device="cuda:0")
    mixer = model.blocks[0].mixers()[0]
    late = SimpleNamespace(decode=False, dtype_is_bf16=dtype == "bfloat16", token_capacity=256, n_seqs=1, context_limit=4096)
    assert mixer.prompt_runs(late, "cuda:0") == (8 if dtype == "bfloat16" else 1)      # (what the test is about)
    early = SimpleNamespace(decode=False, dtype_is_bf16=dtype == "bfloat16", token_capacity=256, n_seqs=1, context_limit=1024)
    assert mixer.prompt_runs(early, "cuda:0") == 1
    engine = bt.Engine(model, max_tokens=4096 + 512)
    gen = torch.Generator().manual_seed(13)
    requests = [torch.randint(0, LONG["vocab_size"], (n,), generator=gen).tolist() for n in (3300, 900)]
    chunks, fed, slots = [256, 70], [0, 0], [engine.open(), engine.open()]
    got, rows = [[], []], [[], []]
    while any(f < len(r) for f, r in zip(fed, requests)):
        live = [i for i in range(2) if fed[i] < len(requests[i])]
        entries = [(slots[i], requests[i][fed[i]:fed[i] + chunks[i]]) for i in live]
        wants = [[0, len(e[1]) // 2, len(e[1]) - 1] for e in entries]
        logits = engine.step(entries, want=wants).clone()
        for n, i in enumerate(live):
            got[i].append(logits[3 * n:3 * n + 3])
            rows[i] += [fed[i] + w for w in wants[n]]
            fed[i] += len(entries[n][1])
    for i, r in enumerate(requests):
        want = plain.forward(r, weights, LONG, rows=rows[i])
        check(torch.cat(got[i]), want, dtype, f"request {i} of {len(r)} tokens in chunks of {chunks[i]}")


SMALL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 12, "n_embd": 768, "n_head": 12,
         "n_inner": 3072, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
         "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
_small = {}


def small_model():
    if not _small:
        holder = tempfile.TemporaryDirectory(prefix="bt_small_")
        weights = bt.write_random_model(holder.name, SMALL, 4)
        _small.update(holder=holder, weights={k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v.float())
                                              for k, v in weights.items()}, models={})
    return _small["holder"].name, _small["weights"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_twelve_layers_of_gpt2_small(dtype):
    """A ragged batch of three prompts in one step, then eight tokens each one by one, through all
    twelve layers of GPT-2 small's sizes: what an error that grows with depth would show."""
    folder, weights = small_model()
    if dtype not in _small["models"]:
        _small["models"][dtype] = bt.load_model(folder, dtype=dtype, device="cuda:0")
    engine = bt.Engine(_small["models"][dtype], max_tokens=2048)
    gen = torch.Generator().manual_seed(9)
    lengths = [1000, 301, 17]
    requests = [torch.randint(0, SMALL["vocab_size"], (n + 8,), generator=gen).tolist() for n in lengths]
    slots = [engine.open() for _ in requests]
    wants = [[0, n // 2, n - 1] for n in lengths]
    rows = [list(w) for w in wants]
    logits = engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, lengths)], want=wants).clone()
    got = [[logits[3 * i:3 * i + 3]] for i in range(3)]
    for t in range(8):
        logits = engine.step([(s, [r[n + t]]) for s, r, n in zip(slots, requests, lengths)]).clone()
        for i, n in enumerate(lengths):
            got[i].append(logits[i:i + 1])
            rows[i].append(n + t)
    for i, request in enumerate(requests):
        check(torch.cat(got[i]), plain.forward(request, weights, SMALL, rows=rows[i]), dtype, f"request {i}")
    for slot in slots:
        engine.close(slot)
