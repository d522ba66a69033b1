"""Guards on speed: they read clocks, so their verdict depends on the machine and on what else runs
on it.  They carry the marker ``perf`` and not ``gpu``: the correctness run (``-m gpu``) leaves them
out, ``pytest -m perf`` on a GPU box runs them, and without a GPU they are skipped."""

import time

import pytest
import torch

pytestmark = [pytest.mark.perf,
              pytest.mark.skipif(not torch.cuda.is_available(), reason="speed is measured on a GPU")]

import burn_transformers_amd as bt  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from model_helpers import model_folder, prompts_for  # noqa: E402

DEV = "cuda:0"


def model_for(name, dtype):
    folder, _, _ = model_folder(name)
    return bt.load_model(folder, dtype=dtype, device=DEV)


def test_host_time_of_a_listed_step_is_a_fraction_of_the_direct_one():
    """What the list is for: the host's share of a step.  Measured without waiting for the GPU
    (the calls only queue work): the same steps issued from Python cost several times more."""
    model = model_for("BW", "bfloat16")
    ids = prompts_for("BW", [64], seed=85)[0]
    seconds = {}
    for programs in (True, False):
        engine = bt.Engine(model, max_tokens=64 * 4, graphs=False, programs=programs)
        slot = engine.open()
        engine.step([(slot, ids)])
        engine.truncate(slot, 0)
        torch.cuda.synchronize()
        started = time.perf_counter()
        for _ in range(20):
            engine.step([(slot, ids)])
            engine.truncate(slot, 0)
        seconds[programs] = (time.perf_counter() - started) / 20
        torch.cuda.synchronize()
    print(f"host time of a 64-token step of a 3-layer model: {seconds[True] * 1e6:.0f} us from a launch list, "
          f"{seconds[False] * 1e6:.0f} us call by call")
    assert seconds[True] < 0.7 * seconds[False]


def test_tile_product_keeps_its_speed_at_the_sizes_it_was_tuned_for():
    """A guard against a change that makes the tile kernel spill its accumulators (an epilogue path
    too many did, once: 75 -> 260 us): 2,048 x 4,800 x 1,600 in bfloat16 takes about 75 us (85 with
    the activation), and the bound here is twice that."""
    m, n, k = 2048, 4800, 1600
    a = torch.randn(m, k, device=DEV).to(torch.bfloat16)
    weights = [(torch.randn(n, k, device=DEV) * 0.02).to(torch.bfloat16) for _ in range(8)]
    bias = torch.randn(n, device=DEV)
    out = torch.empty(m, n, device=DEV, dtype=torch.bfloat16)
    for act in (False, True):
        make = (lambda: K.epilogue_act(out, "gelu_tanh", bias)) if act else (lambda: K.epilogue_store(out, bias))
        K.gemm(a, weights[0], make(), impl="tile")
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(3):
            begin.record()
            for w in weights:
                K.gemm(a, w, make(), impl="tile")
            end.record()
            end.synchronize()
            best = min(best, begin.elapsed_time(end) * 1e3 / len(weights))
        assert best < 170.0, f"the tile product takes {best:.0f} us (activation epilogue: {act})"
