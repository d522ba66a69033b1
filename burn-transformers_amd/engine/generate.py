"""The generation loop above the step function.

Requests (prompts of unequal length) are taken in order and packed into batches that fit the
cache; each batch is prefilled in one step (or in chunks), then decoded one token per step.
A sequence that ends leaves the batch at once and gives its slot back; the next batch uses
the slots again.  One readback per step brings the chosen ids and their log-probabilities to
the host (src/generation/causal.rs:118-211 is the reference's loop; its rows stay in the
batch with a mask, here they leave it).
"""

import math

import torch

from ..cache.ledger import BLOCK
from ..sampling.config import GenerationConfig, GenerationError
from ..sampling.sampler import Sampler
from ..sampling.tracker import GenerationTracker, required_capacity


def _rounded(tokens):
    return (tokens + BLOCK - 1) // BLOCK * BLOCK


def new_token_limits(prompt_lengths, max_new_tokens, total_length=None):
    """New tokens each request may get: max_new_tokens, or fewer where prompt and output together
    would pass ``total_length``."""
    if total_length is None:
        return [max_new_tokens] * len(prompt_lengths)
    for index, length in enumerate(prompt_lengths):
        if length >= total_length:
            raise GenerationError(f"prompt {index} holds {length} tokens already, total_length is {total_length}")
    return [min(max_new_tokens, total_length - length) for length in prompt_lengths]


def plan_batches(prompt_lengths, max_new_tokens, max_tokens, max_slots, sequence_limit, batch_size=None):
    """Splits requests, in order, into batches whose sequences fit the cache together.
    ``max_new_tokens`` is one number or one per request.  Pure bookkeeping; raises if a single
    request cannot fit."""
    batches, current, used = [], [], 0
    limits = max_new_tokens if isinstance(max_new_tokens, (list, tuple)) else [max_new_tokens] * len(prompt_lengths)
    for index, length in enumerate(prompt_lengths):
        if length <= 0:
            raise GenerationError(f"prompt {index} is empty")
        need = required_capacity(length, limits[index])
        if need > sequence_limit:
            raise GenerationError(
                f"prompt {index}: {length} prompt tokens + {limits[index]} new tokens need {need} positions, "
                f"the limit is {sequence_limit}")
        if _rounded(need) > max_tokens:
            raise GenerationError(f"prompt {index} needs {_rounded(need)} cache tokens, the cache holds {max_tokens}")
        full = (batch_size is not None and len(current) >= batch_size) or len(current) >= max_slots
        if current and (full or used + _rounded(need) > max_tokens):
            batches.append(current)
            current, used = [], 0
        current.append(index)
        used += _rounded(need)
    if current:
        batches.append(current)
    return batches


def prefill_chunks(prompt_lengths, chunk):
    """For chunked prefill: a list of steps, each a list of (row, begin, end) token ranges.  Rows
    that have run out of prompt are simply absent from later chunks."""
    if chunk is None:
        return [[(row, 0, n) for row, n in enumerate(prompt_lengths)]]
    if chunk <= 0:
        raise GenerationError("prefill_chunk_size must be greater than zero")
    steps = []
    for begin in range(0, max(prompt_lengths), chunk):
        steps.append([(row, begin, min(begin + chunk, n)) for row, n in enumerate(prompt_lengths) if n > begin])
    return steps


def generate_batch(engine, prompts, config, prefill_chunk=None, on_token=None, limits=None):
    """Runs one batch that starts together to completion; returns its GeneratedSequences.
    ``limits``: new tokens each row may get, where that is less than config.max_new_tokens."""
    tracker = GenerationTracker(config, [len(p) for p in prompts], limits)
    sampler = Sampler(config, len(prompts), engine.device, engine.model.vocab_size, prompts)
    slots = [engine.open() for _ in prompts]
    open_rows = set(range(len(prompts)))
    try:
        logits = torch.empty((len(prompts), engine.model.vocab_size), dtype=torch.float32, device=engine.device)
        for chunk in prefill_chunks([len(p) for p in prompts], prefill_chunk):
            entries = [(slots[row], prompts[row][begin:end]) for row, begin, end in chunk]
            # each row's logits are wanted from the chunk in which its prompt ends
            final = [row for row, _, end in chunk if end == len(prompts[row])]
            want = [[end - begin - 1] if end == len(prompts[row]) else [] for row, begin, end in chunk]
            chunk_logits = engine.step(entries, want)
            if final:
                logits.index_copy_(0, torch.tensor(final, device=engine.device), chunk_logits)
        live = list(range(len(prompts)))
        if sampler.pipelined:
            _decode_ahead(engine, sampler, tracker, slots, open_rows, logits, live, on_token)
            return tracker.sequences
        while True:
            ids, logps = sampler.select(logits, live)
            next_live, next_entries = [], []
            for row, token, logp in zip(live, ids, logps):
                if not math.isfinite(logp):
                    raise GenerationError(f"row {row}: the selected token has a non-finite log-probability")
                reason = tracker.push(row, token, logp)
                if on_token is not None:
                    on_token(row, token, logp, reason)
                if reason is None:
                    next_live.append(row)
                    next_entries.append((slots[row], [token]))
                else:                                   # the sequence leaves the batch; its slot is free again
                    engine.close(slots[row])
                    open_rows.discard(row)
            if not next_live:
                break
            live = next_live
            logits = engine.step(next_entries)
    finally:
        for row in open_rows:
            engine.close(slots[row])
    return tracker.sequences


def select_and_step_ahead(engine, sampler, slots, logits, live, ahead):
    """One turn of the decode pipeline, with the host one step behind the GPU: starts the selection
    of one token for every row of ``live`` from ``logits``; feeds the rows of ``ahead`` (those of
    ``live`` that go on unless this very token stops them, in the same order) their tokens straight
    from the GPU (``Engine.step(device_tokens=...)``); only then waits for the selection's ids to
    reach the host, while that step already runs.  Returns (ids, log-probabilities, the logits of
    the step that was started for ``ahead``, or None if no row goes on).  The generation loop and
    the benchmark both decode through this function."""
    sampler.launch(logits, live)
    next_logits = None
    if ahead:
        tokens = sampler.device_ids(len(live))
        if len(ahead) != len(live):
            going = set(ahead)
            places = [i for i, row in enumerate(live) if row in going]
            tokens = tokens[torch.tensor(places, device=engine.device)]
        next_logits = engine.step([(slots[row], [0]) for row in ahead], device_tokens=tokens)
    ids, logps = sampler.result()
    return ids, logps, next_logits


def _decode_ahead(engine, sampler, tracker, slots, open_rows, logits, live, on_token):
    """The decode loop with the host one step behind the GPU (``select_and_step_ahead``): the host's
    own work (stop rules, the next step's tables) costs the GPU no idle time.  A row whose token
    turns out to end it (end-of-sequence, a stop sequence) has then been fed once too often: that
    position goes with the row's slot.  Rows that end by their length are known beforehand and are
    not fed.  Tokens, log-probabilities and finish reasons are those of the loop that waits for
    every token up to rounding: a row that its token ends stays in the batch for one more step,
    and the number of rows chooses the kernels of a step, so in bfloat16 the other rows' logits of
    that one step may round differently than they would without it, and a near-tie may then choose
    another token."""
    device = engine.device
    while True:
        # rows that go on unless this very token stops them
        ahead = [row for row in live if len(tracker.sequences[row].token_ids) + 1 < tracker.limit(row)]
        ids, logps, next_logits = select_and_step_ahead(engine, sampler, slots, logits, live, ahead)
        next_live = []
        for row, token, logp in zip(live, ids, logps):
            if not math.isfinite(logp):
                raise GenerationError(f"row {row}: the selected token has a non-finite log-probability")
            reason = tracker.push(row, token, logp)
            if on_token is not None:
                on_token(row, token, logp, reason)
            if reason is None:
                next_live.append(row)
            else:                                   # the sequence leaves the batch; its slot is free again
                engine.close(slots[row])
                open_rows.discard(row)
        if not next_live:
            return
        if len(next_live) != len(ahead):            # a token ended its row: that row's logits are dropped
            kept = set(next_live)
            places = [i for i, row in enumerate(ahead) if row in kept]
            next_logits = next_logits[torch.tensor(places, device=device)]
        logits, live = next_logits, next_live


def generate(engine, prompts, config=None, prefill_chunk=None, batch_size=None, on_token=None, total_length=None):
    """Generates for every prompt (lists of token ids); returns GeneratedSequences in order.
    With ``total_length`` a sequence also ends (Length) when prompt and output together hold that
    many tokens, so unequal prompts can all be grown to the model's position limit."""
    config = config or GenerationConfig()
    config.validate(engine.model.vocab_size)
    prompts = [list(p) for p in prompts]
    if not prompts:
        raise GenerationError("no prompts")
    limit = min(engine.model.max_positions, engine.cache.max_sequence_length)
    limits = new_token_limits([len(p) for p in prompts], config.max_new_tokens, total_length)
    batches = plan_batches([len(p) for p in prompts], limits, engine.cache.max_tokens,
                           engine.cache.max_slots, limit, batch_size)
    results = [None] * len(prompts)
    for batch in batches:
        callback = None
        if on_token is not None:
            callback = lambda row, token, logp, reason, batch=batch: on_token(batch[row], token, logp, reason)
        for index, sequence in zip(batch, generate_batch(engine, [prompts[i] for i in batch], config,
                                                         prefill_chunk, callback, [limits[i] for i in batch])):
            results[index] = sequence
    return results
