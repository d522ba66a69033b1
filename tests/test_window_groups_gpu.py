"""Groups of layers with different needs: layers that read every key beside layers that read a
window of the latest keys.  Each group has storage, free blocks and block tables of its own, and
the windowed group gives a sequence's blocks back as the window moves past them, while the
sequence is still growing.

GPT-2 has no windows; the family here is GPT-2's plan with a window written into some layers'
attention, registered from this file alone."""

from dataclasses import dataclass
from typing import Tuple

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from burn_transformers_amd.architectures import gpt2  # noqa: E402
from burn_transformers_amd.cache.ledger import RELEASED  # noqa: E402
from burn_transformers_amd.config.gpt2 import GPT2Config  # noqa: E402
from model_helpers import tolerance  # noqa: E402


@dataclass(frozen=True)
class WindowedConfig:
    base: GPT2Config
    windows: Tuple[int, ...]

    @classmethod
    def from_dict(cls, data):
        base = GPT2Config.from_dict({k: v for k, v in data.items() if k not in ("windows", "architectures")})
        windows = tuple(data["windows"])
        assert len(windows) == base.n_layer
        return cls(base, windows)

    def to_dict(self):
        return dict(self.base.to_dict(), architectures=["ToyWindowedLM"], windows=list(self.windows))


def windowed_plan(config):
    plan = gpt2.plan(config.base)
    for layer, window in zip(plan.layers, config.windows):
        layer.parts["mixer"].params["window"] = window
    return plan


def reference(ids, w, config):
    """Whole sequence in float64 with the plain implementation's parts, each layer with its window."""
    c = config.base
    w = {k: v.double() for k, v in w.items()}
    ids = torch.as_tensor(ids)
    x = plain.embed(ids, torch.arange(len(ids)), w["wte.weight"], w["wpe.weight"])
    for i, window in enumerate(config.windows):
        p = f"h.{i}."
        scale = plain.attention_scale(c.head_size, i, True, c.scale_attn_by_inverse_layer_idx)
        h = plain.layer_norm(x, w[p + "ln_1.weight"], w[p + "ln_1.bias"], c.layer_norm_epsilon)
        x = x + plain.self_attention(h, w, p + "attn.", c.n_head, scale, True, window or None)
        h = plain.layer_norm(x, w[p + "ln_2.weight"], w[p + "ln_2.bias"], c.layer_norm_epsilon)
        x = x + plain.mlp(h, w[p + "mlp.c_fc.weight"], w[p + "mlp.c_fc.bias"], w[p + "mlp.c_proj.weight"],
                          w[p + "mlp.c_proj.bias"], c.activation_function)
    x = plain.layer_norm(x, w["ln_f.weight"], w["ln_f.bias"], c.layer_norm_epsilon)
    return x @ w["wte.weight"].t()


CONFIG = {"architectures": ["ToyWindowedLM"], "model_type": "gpt2", "n_layer": 4, "n_embd": 64, "n_head": 2,
          "n_inner": 96, "vocab_size": 211, "n_positions": 640, "activation_function": "gelu_new",
          "layer_norm_epsilon": 1e-5, "windows": [0, 70, 200, 70]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_with_windows_give_blocks_back_and_read_nothing_that_is_gone(dtype):
    bt.register_family(bt.Family("toy_windowed", ("ToyWindowedLM",), (), WindowedConfig, windowed_plan,
                                 lambda c: gpt2.contract(c.base), lambda c, g: gpt2.init(c.base, g)))
    try:
        config = WindowedConfig.from_dict(CONFIG)
        _, tensors = bt.random_tensors(CONFIG, 9)
        tensors = {k: (v * 5.0 if v.dim() == 2 else v).to(torch.bfloat16).float() for k, v in tensors.items()}
        model = bt.model_from_tensors(CONFIG, tensors, dtype=dtype, device="cuda:0")
        engine = bt.Engine(model, max_tokens=64 * 17, graphs="always")
        cache, ledger = engine.cache, engine.cache.ledger
        # three groups: every key (layer 0), the last 70 (layers 1 and 3), the last 200 (layer 2)
        assert sorted(ledger.windows) == [0, 70, 200] and [g.entries for g in cache.kv_groups] == [1, 2, 1]
        group = {w: ledger.windows.index(w) for w in (0, 70, 200)}
        # everything in the cache is poison, and block 0 of every group (what a released block's place
        # in a table names) stays poison: a dummy sequence holds it and never writes to it
        for g in cache.kv_groups:
            g.keys.fill_(float("nan"))
            g.values.fill_(float("nan"))
        dummy = engine.open()
        ledger.reserve(dummy, 1)
        assert all(ledger.held_blocks[g][dummy] == [0] for g in range(3))

        gen = torch.Generator().manual_seed(10)
        requests = [torch.randint(0, 211, (n,), generator=gen).tolist() for n in (600, 150)]
        wants = [reference(r, tensors, config) for r in requests]
        slots = [engine.open(), engine.open()]
        got, fed = [[], []], [0, 0]
        schedule = [(150, 100)] + [(1, 1)] * 20 + [(130, 30)] + [(1, 0)] * 40 + [(200, 0), (1, 0), (59, 0)]
        for counts in schedule:
            live = [i for i in range(2) if counts[i] and fed[i] < len(requests[i])]
            entries = [(slots[i], requests[i][fed[i]:fed[i] + counts[i]]) for i in live]
            logits = engine.step(entries, want=[list(range(len(e[1]))) for e in entries]).clone()
            at = 0
            for i, e in zip(live, entries):
                got[i].append(logits[at:at + len(e[1])])
                at += len(e[1])
                fed[i] += len(e[1])
            ledger.check()
            length = engine.length(slots[0])
            for window in (70, 200):           # blocks wholly behind the window are gone, the others are there
                held = ledger.held_blocks[group[window]][slots[0]]
                first = max(0, length - window + 1) // 64
                assert held[:first] == [RELEASED] * first and RELEASED not in held[first:]
            assert RELEASED not in ledger.held_blocks[group[0]][slots[0]]
        assert fed == [600, 150] and engine.graph_replays > 30
        # 600 tokens are 10 blocks where every key is kept, 2 where the last 70 are, 4 where the last 200 are
        assert [sum(b != RELEASED for b in ledger.held_blocks[group[w]][slots[0]]) for w in (0, 70, 200)] == [10, 2, 4]
        for i, want in enumerate(wants):
            rows = torch.cat(got[i]).cpu().double()
            assert torch.isfinite(rows).all()
            error = float((rows - want).abs().max())
            assert error <= tolerance(dtype, want), f"request {i}: {error} > {tolerance(dtype, want)}"
        # a sequence that starts now takes blocks the window gave back, and is right as well
        extra = engine.open()
        logits = engine.step([(extra, requests[1][:100])], want=[list(range(100))])
        error = float((logits.cpu().double() - wants[1][:100]).abs().max())
        assert error <= tolerance(dtype, wants[1]), f"a later sequence: {error}"
        with pytest.raises(ValueError, match="window of"):
            engine.truncate(slots[0], 300)
        engine.reset()
        ledger.check()
        assert all(f.available() == f.count for f in ledger.blocks)
    finally:
        bt.unregister_family("toy_windowed")
