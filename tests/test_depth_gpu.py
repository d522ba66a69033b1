"""The engine at the depth and sizes the benchmark runs at, against the plain implementation.

GPT-2 XL's configuration with all 48 layers (width 1600, 25 heads of 64, inner width 6400,
50,257 tokens, 1,024 positions), random weights, in float32 and in bfloat16: a request whole,
the same request with its last 32 tokens one by one, and two batches of unequal lengths after
one another, the second in the slots of the first.  An error that grows with depth (the order of
the residual sums, a partial sum added twice, bfloat16 rounding of the stream) shows here and
not at two layers.  Queries and keys are scaled up as in ``test_real_sizes_gpu.py`` so that
attention is peaked.

Then GPT-2 small's configuration in float32 through ``bin/trace_run``: a batch of 16 prompts of
unequal lengths between 1 and 1,000 tokens in one step, then some tokens each one by one."""

import json
import os
import subprocess
import sys
import tempfile

import numpy as np
import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.slow]

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402

XL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 48, "n_embd": 1600, "n_head": 25,
      "n_inner": 6400, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
      "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
SHARPEN = 2.5
_xl = {}


def xl_weights():
    """float32 weights whose matrices are bfloat16 values (both precisions then hold the same
    numbers), and the same in float64 for the plain implementation."""
    if not _xl:
        print("[depth] drawing 1.56e9 weights", flush=True)
        _, tensors = bt.random_tensors(XL, 11)
        d = XL["n_embd"]
        for layer in range(XL["n_layer"]):
            tensors[f"h.{layer}.attn.c_attn.weight"][:, :2 * d] *= SHARPEN
            tensors[f"h.{layer}.attn.c_attn.bias"][:2 * d] *= SHARPEN
        tensors = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v.float()) for k, v in tensors.items()}
        _xl.update(tensors=tensors, wide={k: v.double() for k, v in tensors.items()}, models={}, oracle={})
    return _xl["tensors"]


def xl_engine(dtype, max_tokens):
    tensors = xl_weights()
    if dtype not in _xl["models"]:
        print(f"[depth] building the {dtype} model", flush=True)
        _xl["models"][dtype] = bt.model_from_tensors(XL, tensors, dtype=dtype, device="cuda:0")
    return bt.Engine(_xl["models"][dtype], max_tokens=max_tokens)


def request(length, seed):
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, XL["vocab_size"], (length,), generator=gen).tolist()


def oracle(ids):
    """float64 logits of every position of the request (kept: both precisions ask for the same)."""
    xl_weights()
    key = tuple(ids)
    if key not in _xl["oracle"]:
        print(f"[depth] plain forward of {len(ids)} tokens through 48 layers", flush=True)
        _xl["oracle"][key] = plain.forward(ids, _xl["wide"], XL)
    return _xl["oracle"][key]


# float32: the reference's own acceptance bound for logits, 1e-4 + 1e-5 |ref|, element by element
# (src/models/gpt2/README.md:71-73).  bfloat16: every activation between two kernels is rounded to 8
# bits (relative 2^-9), 48 layers of four such roundings each add up in the float32 stream like a
# random walk; measured here: 1.1e-2 of the largest logit at worst (rows of 96 positions, three
# requests).  The bound is twice that.
def check(got, want, dtype, what):
    got = got.detach().cpu().double()
    assert torch.isfinite(got).all(), what
    error = (got - want).abs()
    if dtype == "float32":
        excess = float((error - (1e-4 + 1e-5 * want.abs())).max())
        print(f"[depth] {what} ({dtype}): max error {float(error.max()):.3g}", flush=True)
        assert excess <= 0, f"{what}: an element is {excess} beyond 1e-4 + 1e-5 |ref| (max error {float(error.max())})"
    else:
        relative = float(error.max() / want.abs().max())
        print(f"[depth] {what} ({dtype}): max error {float(error.max()):.3g}, {relative:.3g} of the largest logit", flush=True)
        assert relative <= BF16_BOUND, f"{what}: error {relative} of the largest logit > {BF16_BOUND}"
        # and the decisions agree: the plain implementation's best token is among the engine's best few
        top = want.argmax(-1)
        rank = (got > got.gather(1, top[:, None])).sum(-1)
        assert int(rank.max()) < 50, f"{what}: the reference's best token has rank {int(rank.max())}"


BF16_BOUND = 2.2e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_48_layers_whole_then_tail_one_by_one(dtype):
    ids = request(96, seed=1)
    want = oracle(ids)
    engine = xl_engine(dtype, max_tokens=1024)
    slot = engine.open()
    logits = engine.step([(slot, ids)], want=[list(range(len(ids)))])
    check(logits, want, dtype, "request of 96 whole")
    engine.close(slot)
    slot = engine.open()
    got = [engine.step([(slot, ids[:64])], want=[list(range(64))]).clone()]
    for t in range(64, 96):
        got.append(engine.step([(slot, [ids[t]])]).clone())
    check(torch.cat(got), want, dtype, "the same with its last 32 tokens one by one")
    # the engine chose for itself how the repeating decode shape runs (from its launch list or from
    # a graph, by what it measured on this machine): either way the steps did not come from Python
    assert engine.graph_replays + engine.program_runs >= 28
    engine.close(slot)
    engine.cache.ledger.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_48_layers_unequal_batches_one_after_another(dtype):
    engine = xl_engine(dtype, max_tokens=64 * 5)
    first = request(96, seed=1)
    batches = [([request(74, seed=2), request(22, seed=3), first[:39]], [70, 20, 33]),
               ([request(43, seed=4), first[:80]], [40, 65])]
    seen = []
    for b, (requests, prompts) in enumerate(batches):
        slots = [engine.open() for _ in requests]
        seen.append(list(slots))
        logits = engine.step([(s, r[:n]) for s, r, n in zip(slots, requests, prompts)],
                             want=[list(range(n)) for n in prompts]).clone()
        got, at = [], 0
        for n in prompts:
            got.append([logits[at:at + n]])
            at += n
        live, position = list(range(len(requests))), list(prompts)
        while live:
            logits = engine.step([(slots[i], [requests[i][position[i]]]) for i in live]).clone()
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                position[i] += 1
            for i in [i for i in live if position[i] >= len(requests[i])]:
                engine.close(slots[i])               # ends earlier than the others
                live.remove(i)
        for i, r in enumerate(requests):
            want = oracle(first)[:len(r)] if r == first[:len(r)] else oracle(r)
            check(torch.cat(got[i]), want, dtype, f"batch {b} request {i} ({len(r)} tokens)")
        engine.cache.ledger.check()
    assert set(seen[0]) & set(seen[1]), "slots were not used again"


# --- GPT-2 small, float32, a batch of 16 unequal prompts through bin/trace_run -------------------

SMALL = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 12, "n_embd": 768, "n_head": 12,
         "n_inner": 3072, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
         "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DECODED = 6


def test_sixteen_unequal_prompts_of_gpt2_small_through_trace_run(tmp_path):
    """Lengths uniform in [1, 1000] (the shortest and the longest made sure of), all prompts in one
    step, then ``DECODED`` tokens each one by one, or fewer where a request ends earlier; logits at
    each prompt's first, middle and last place and at every decoded token.  The plain
    implementation checks six of the sixteen: the shortest, the longest and four between."""
    gen = torch.Generator().manual_seed(21)
    lengths = torch.randint(1, 1001, (16,), generator=gen).tolist()
    lengths[3], lengths[12] = 1, 1000
    extra = [DECODED - (i % 3) for i in range(16)]
    requests = [torch.randint(0, SMALL["vocab_size"], (n + e,), generator=gen).tolist() for n, e in zip(lengths, extra)]
    holder = tempfile.TemporaryDirectory(prefix="bt_small_trace_")
    weights = bt.write_random_model(holder.name, SMALL, 4)
    weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}       # as stored
    places = [sorted({0, n // 2, n - 1}) for n in lengths]
    steps = [{"step": 0, "entries": [{"id": f"r{i}", "tokens": r[:n], "want": places[i]}
                                     for i, (r, n) in enumerate(zip(requests, lengths))], "end": []}]
    rows = {i: [(0, sum(len(p) for p in places[:i]), len(places[i]))] for i in range(16)}
    for t in range(DECODED):
        live = [i for i in range(16) if t < extra[i]]
        steps.append({"step": t + 1, "entries": [{"id": f"r{i}", "tokens": [requests[i][lengths[i] + t]], "want": [0]}
                                                 for i in live],
                      "end": [f"r{i}" for i in live if t + 1 == extra[i]]})
        for row, i in enumerate(live):
            rows[i].append((t + 1, row, 1))
    budget = sum((len(r) + 63) // 64 * 64 for r in requests)
    out_dir = tmp_path / "out"
    lines = "".join(json.dumps(s) + "\n" for s in steps)
    result = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", holder.name,
                             "--dtype", "float32", "--out", str(out_dir), "--max-tokens", str(budget)],
                            input=lines, capture_output=True, text=True, timeout=600)
    assert result.returncode == 0, result.stderr[-2000:]
    assert result.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    out = {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        data = np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4")
        out[s["step"]] = torch.from_numpy(data.reshape(wanted, SMALL["vocab_size"]).copy())
    order = sorted(range(16), key=lambda i: lengths[i])
    for i in [order[0], order[4], order[8], order[11], order[14], order[15]]:
        n = lengths[i]
        got = torch.cat([out[s][row:row + count] for s, row, count in rows[i]]).double()
        want = plain.forward(requests[i], weights, SMALL, rows=places[i] + list(range(n, n + extra[i])))
        error = (got - want).abs()
        excess = float((error - (1e-4 + 1e-5 * want.abs())).max())
        print(f"[depth] trace_run request {i} ({n} + {extra[i]} tokens): max error {float(error.max()):.3g}", flush=True)
        assert excess <= 0, f"request {i} of {n} tokens: {excess} beyond 1e-4 + 1e-5 |ref|"
