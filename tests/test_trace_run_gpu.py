"""bin/trace_run as a user runs it: a subprocess fed JSON lines, whose logit files are compared
with the plain implementation for every way of cutting the same requests."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from model_helpers import CONFIGS, model_folder, plain_logits, prompts_for, tolerance  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def replay(name, dtype, steps, out_dir, max_tokens):
    folder, _, _ = model_folder(name)
    lines = "".join(json.dumps(s) + "\n" for s in steps)
    result = subprocess.run([sys.executable, TRACE_RUN, "--model", folder, "--dtype", dtype, "--out", str(out_dir),
                             "--max-tokens", str(max_tokens)], input=lines, capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr[-2000:]
    assert result.stdout.split("\n")[:len(steps)] == [f"done {s['step']}" for s in steps]
    vocab = CONFIGS[name][0]["vocab_size"]
    out = {}
    for s in steps:
        path = os.path.join(out_dir, f"{s['step']}.f32")
        wanted = sum(len(e.get("want", [])) for e in s["entries"])
        assert os.path.exists(path) == (wanted > 0)
        if wanted:
            out[s["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy())
    return out


def whole_trace(requests):
    """Each request alone and whole, one after another (slots are used again)."""
    return [{"step": i, "entries": [{"id": f"r{i}", "tokens": r, "want": list(range(len(r)))}], "end": [f"r{i}"]}
            for i, r in enumerate(requests)]


def tail_trace(request, tail=32):
    head = len(request) - tail
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": request[:head], "want": list(range(head))}], "end": []}]
    for i in range(tail):
        steps.append({"step": i + 1, "entries": [{"id": "a", "tokens": [request[head + i]], "want": [0]}],
                      "end": ["a"] if i == tail - 1 else []})
    return steps


def batched_trace(batches, prompt_lengths):
    """Batches of unequal lengths that start together, go on by one token per step, and whose
    shorter requests end earlier; one batch after another.  Returns (steps, where) with
    where[(batch, request)] = list of (step, first row, rows) pieces in order of position."""
    steps, where, number = [], {}, 0
    for b, (requests, prompts) in enumerate(zip(batches, prompt_lengths)):
        ids = [f"b{b}r{i}" for i in range(len(requests))]
        entries = [{"id": ids[i], "tokens": r[:n], "want": list(range(n))} for i, (r, n) in enumerate(zip(requests, prompts))]
        at = 0
        for i, n in enumerate(prompts):
            where[(b, i)] = [(number, at, n)]
            at += n
        done = [ids[i] for i, (r, n) in enumerate(zip(requests, prompts)) if n == len(r)]
        steps.append({"step": number, "entries": entries, "end": done})
        number += 1
        position = list(prompts)
        live = [i for i in range(len(requests)) if position[i] < len(requests[i])]
        while live:
            entries = [{"id": ids[i], "tokens": [requests[i][position[i]]], "want": [0]} for i in live]
            for row, i in enumerate(live):
                where[(b, i)].append((number, row, 1))
                position[i] += 1
            done = [ids[i] for i in live if position[i] == len(requests[i])]
            steps.append({"step": number, "entries": entries, "end": done})
            live = [i for i in live if position[i] < len(requests[i])]
            number += 1
    return steps, where


def compare(name, dtype, got, want, what):
    error = float((got.double() - want).abs().max())
    assert error <= tolerance(dtype, want), f"{what}: {error} > {tolerance(dtype, want)}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths", [("A", [40, 128, 65]), ("BW", [33, 192, 100])])
def test_replay_whole_tail_and_batches(name, dtype, lengths, tmp_path):
    requests = prompts_for(name, lengths, seed=50)
    reference = [plain_logits(name, r) for r in requests]
    limit = CONFIGS[name][0]["n_positions"]

    out = replay(name, dtype, whole_trace(requests), tmp_path / "whole", max_tokens=limit)
    for i, want in enumerate(reference):
        compare(name, dtype, out[i], want, f"whole request {i}")

    for i, r in enumerate(requests):
        out = replay(name, dtype, tail_trace(r), tmp_path / f"tail{i}", max_tokens=limit)
        got = torch.cat([out[s] for s in range(33)])
        compare(name, dtype, got, reference[i], f"last 32 tokens of request {i} one by one")

    more = prompts_for(name, [7, 70, 64, 1], seed=51)
    batches = [requests, more, [requests[2], more[1]]]
    prompt_lengths = [[n - 9 - 3 * i for i, n in enumerate(lengths)], [3, 61, 64, 1], [1, 2]]
    steps, where = batched_trace(batches, prompt_lengths)
    budget = max(sum((len(r) + 63) // 64 * 64 for r in batch) for batch in batches)
    out = replay(name, dtype, steps, tmp_path / "batches", max_tokens=budget)
    for (b, i), pieces in where.items():
        got = torch.cat([out[s][row:row + n] for s, row, n in pieces])
        compare(name, dtype, got, plain_logits(name, batches[b][i]), f"batch {b} request {i}")


def test_replay_steps_without_wanted_places_write_nothing(tmp_path):
    r = prompts_for("A", [50], seed=52)[0]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": r[:30], "want": []},
                                     {"id": "idle", "tokens": [], "want": []}], "end": []},      # an entry that brings nothing
             {"step": 1, "entries": [{"id": "x", "tokens": r[30:], "want": [19]}], "end": ["x", "idle"]}]
    out = replay("A", "float32", steps, tmp_path, max_tokens=64)
    assert list(out) == [1]
    compare("A", "float32", out[1], plain_logits("A", r)[-1:], "cache filled by a step nobody read")
