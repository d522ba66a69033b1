"""Builds a step by hand, without an engine, for tests of single parts."""

import numpy as np
import torch

from burn_transformers_amd.engine.step import BufferPool, Step, StepPlan


def make_step(dtype, counts, starts=None, ids=None, wanted=None, cache=None, slots=None, pool=None,
              device="cuda:0"):
    n = len(counts)
    starts = list(starts) if starts is not None else [0] * n
    slots = list(slots) if slots is not None else list(range(n))
    total = int(sum(counts))
    ids = np.asarray(ids if ids is not None else np.zeros(total), dtype=np.int64)
    wanted = list(wanted) if wanted is not None else [int(x) - 1 for x in np.cumsum(counts)]
    if cache is not None:
        rows, max_blocks = cache.block_rows(slots), cache.max_blocks
    else:
        rows, max_blocks = [[[] for _ in slots]], 1
    plan = StepPlan(slots, starts, list(counts), ids, wanted, rows, max_blocks)
    meta = torch.from_numpy(plan.host).to(device)
    return Step(plan.layout, meta, pool or BufferPool(torch.device(device)), dtype, plan)
