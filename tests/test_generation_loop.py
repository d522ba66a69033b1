"""The generation loop's decisions: stop rules, batching, chunking (no GPU)."""

import pytest

import burn_transformers_amd as bt
from burn_transformers_amd.engine.generate import new_token_limits, plan_batches, prefill_chunks
from burn_transformers_amd.sampling.tracker import (GenerationTracker, required_capacity,
                                                    stop_decision)


def test_generation_config_names_the_first_invalid_field():
    """src/generation.rs:278-405: ranges of every control, checked in float32."""
    bt.GenerationConfig().validate(100)
    bt.GenerationConfig(strategy="sample", top_k=100, top_p=1.0, min_p=0.0, repetition_penalty=1.3, presence_penalty=-2.0,
                        frequency_penalty=0.5, no_repeat_ngram_size=3, logit_bias={99: -5.0},
                        additive_penalty_scope="prompt_and_generated").validate(100)
    cases = [(dict(max_new_tokens=0), "max_new_tokens"), (dict(min_new_tokens=9, max_new_tokens=3), "min_new_tokens"),
             (dict(strategy="beam"), "strategy"), (dict(temperature=0.0), "temperature"),
             (dict(temperature=float("inf")), "temperature"), (dict(temperature=1e-46), "temperature"),
             (dict(eos_token_ids=[100]), "special token 100"), (dict(pad_token_id=-1), "special token -1"),
             (dict(stop_sequences=[[]]), "stop sequences must not be empty"),
             (dict(stop_sequences=[[1, 200]]), "special token 200"),
             (dict(top_k=0), "top_k"), (dict(top_k=101), "top_k"), (dict(top_p=0.0), "top_p"), (dict(top_p=1.5), "top_p"),
             (dict(min_p=-0.1), "min_p"), (dict(min_p=1.1), "min_p"),
             (dict(repetition_penalty=0.0), "repetition_penalty"), (dict(repetition_penalty=1e39), "repetition_penalty"),
             (dict(presence_penalty=float("nan")), "presence_penalty"), (dict(frequency_penalty=1e39), "frequency_penalty"),
             (dict(additive_penalty_scope="prompt"), "additive_penalty_scope"),
             (dict(no_repeat_ngram_size=-1), "no_repeat_ngram_size"),
             (dict(logit_bias={100: 1.0}), "logit_bias token 100"), (dict(logit_bias={3: float("inf")}), "logit_bias for token 3"),
             # the first invalid field in the reference's order is the one that is named
             (dict(temperature=0.0, top_k=0), "temperature"), (dict(top_k=0, repetition_penalty=0.0), "top_k")]
    for fields, name in cases:
        with pytest.raises(bt.GenerationError, match=name):
            bt.GenerationConfig(**fields).validate(100)
    with pytest.raises(bt.GenerationError, match="vocabulary_size"):
        bt.GenerationConfig().validate(0)


def test_which_configurations_process_the_logits():
    plain = bt.GenerationConfig()
    assert not plain.processes_logits(100) and not plain.counts_all and not plain.counts_generated
    assert not bt.GenerationConfig(strategy="sample", temperature=0.5, top_k=100, top_p=1.0, min_p=0.0).processes_logits(100)
    assert not bt.GenerationConfig(top_k=5, top_p=0.5).processes_logits(100)          # greedy ignores the warpers
    assert bt.GenerationConfig(strategy="sample", top_k=5).processes_logits(100)
    assert bt.GenerationConfig(min_new_tokens=2, eos_token_ids=[1]).processes_logits(100)
    assert not bt.GenerationConfig(min_new_tokens=2).processes_logits(100)
    rep = bt.GenerationConfig(repetition_penalty=1.2)
    assert rep.counts_all and not rep.counts_generated and rep.adjusts_logits
    freq = bt.GenerationConfig(frequency_penalty=0.1)
    assert freq.counts_generated and not freq.counts_all
    assert bt.GenerationConfig(presence_penalty=0.1, additive_penalty_scope="prompt_and_generated").counts_all


def test_ngram_index_bans_what_followed_the_same_prefix():
    """src/generation/ngram.rs:1-12: the index against a direct search of the row."""
    import random
    import plain_gpt2 as plain
    from burn_transformers_amd.sampling.history import NgramIndex
    rng = random.Random(0)
    for size in (1, 2, 3, 4):
        index, tokens = NgramIndex(size), []
        assert index.banned() == plain.banned_by_ngrams(tokens, size)
        for _ in range(60):
            token = rng.randrange(4)
            tokens.append(token)
            index.push(token)
            assert index.banned() == plain.banned_by_ngrams(tokens, size), (size, tokens)
    assert plain.banned_by_ngrams([1, 2, 3, 1, 2], 3) == [3]          # 1 2 -> 3 was seen
    assert plain.banned_by_ngrams([1, 2, 3, 1, 2], 2) == [3]          # 2 -> 3
    assert plain.banned_by_ngrams([5, 6, 5], 1) == [5, 6]             # nothing may repeat
    assert plain.banned_by_ngrams([5], 3) == []                       # too short for a prefix of two


def test_plain_truncation_rules():
    """Pins of the plain filters on cases worked by hand (src/generation.rs:1189-1253)."""
    import math
    import torch
    import plain_gpt2 as plain
    z = torch.tensor([1.0, 3.0, 2.0, 3.0, 0.0, -1.0], dtype=torch.float64)
    kept = lambda t: [i for i, v in enumerate(t.tolist()) if v != -math.inf]
    assert kept(plain.filter_top_k(z, 1)) == [1, 3]                   # ties with the boundary survive
    assert kept(plain.filter_top_k(z, 3)) == [1, 2, 3]
    p = torch.softmax(z, -1)
    # ranked 1, 3, 2, 0, 4, 5: an item survives when the mass before it is below p
    assert kept(plain.filter_top_p(z, float(p[1]) * 0.5)) == [1]
    assert kept(plain.filter_top_p(z, float(p[1]) + 1e-9)) == [1, 3]
    assert kept(plain.filter_top_p(z, float(p[1] + p[3] + p[2]) + 1e-9)) == [0, 1, 2, 3]
    assert kept(plain.filter_min_p(z, math.exp(-1.0) - 1e-9)) == [1, 2, 3]     # z >= 3 - 1
    assert kept(plain.filter_min_p(z, math.exp(-1.0) + 1e-9)) == [1, 3]
    assert kept(plain.truncate(z, top_k=6, top_p=1.0, min_p=0.0)) == [0, 1, 2, 3, 4, 5]
    # processing order: bias before the repetition penalty, ban last
    counts = torch.tensor([1, 0, 0, 0, 0, 2])
    out = plain.process_logits(z, sampling=True, temperature=2.0, logit_bias={0: 1.0}, repetition_penalty=2.0,
                               presence_penalty=0.5, frequency_penalty=0.25, seen_counts=counts, additive_counts=counts,
                               banned=[4])
    assert out.tolist() == [((1.0 + 1.0) / 2.0 - 0.25 - 0.5) / 2.0, 1.5, 1.0, 1.5, -math.inf, (-1.0 * 2.0 - 0.5 - 0.5) / 2.0]


def test_end_of_sequence_beats_stop_sequence_beats_length():
    """src/generation/bookkeeping.rs:246-296."""
    cfg = bt.GenerationConfig(max_new_tokens=3, eos_token_ids=[9], stop_sequences=[[5, 9], [9]])
    assert stop_decision(cfg, [1]) is None
    reason = stop_decision(cfg, [1, 5, 9])             # all three rules fire: end-of-sequence wins
    assert reason.kind == "eos" and reason.token_id == 9
    cfg = bt.GenerationConfig(max_new_tokens=3, stop_sequences=[[9], [5, 9], [1, 5, 9], [5, 9]])
    reason = stop_decision(cfg, [1, 5, 9])             # the longest suffix wins
    assert (reason.kind, reason.index, reason.length) == ("stop", 2, 3)
    cfg = bt.GenerationConfig(max_new_tokens=3, stop_sequences=[[5, 9], [5, 9]])
    assert stop_decision(cfg, [0, 5, 9]).index == 0    # ties go to the first configured
    assert stop_decision(bt.GenerationConfig(max_new_tokens=3), [4, 4, 4]).kind == "length"


def test_min_new_tokens_suppresses_early_stops():
    cfg = bt.GenerationConfig(max_new_tokens=5, min_new_tokens=3, eos_token_ids=[9], stop_sequences=[[7]])
    assert stop_decision(cfg, [9]) is None and stop_decision(cfg, [9, 7]) is None
    assert stop_decision(cfg, [9, 7, 9]).kind == "eos"
    assert stop_decision(cfg, [9, 9, 7]).kind == "stop"


def test_tracker_keeps_the_terminal_token_and_refuses_finished_rows():
    cfg = bt.GenerationConfig(max_new_tokens=4, eos_token_ids=[2])
    tracker = GenerationTracker(cfg, [3, 5])
    assert tracker.push(0, 7, -0.5) is None
    assert tracker.push(1, 2, -0.1).kind == "eos"       # emitted, then finished
    assert tracker.sequences[1].token_ids == [2] and tracker.finished(1) and tracker.live_rows() == [0]
    with pytest.raises(RuntimeError, match="already finished"):
        tracker.push(1, 3, 0.0)
    for token in (8, 8):
        assert tracker.push(0, token, -1.0) is None
    assert tracker.push(0, 8, -1.0).kind == "length" and tracker.all_finished()
    assert tracker.sequences[0].prompt_length == 3 and len(tracker.sequences[0].log_probabilities) == 4


def test_required_capacity_leaves_out_the_last_token():
    """src/generation/bookkeeping.rs:736-747."""
    assert required_capacity(10, 1) == 10 and required_capacity(10, 6) == 15


def test_batches_fit_the_cache_and_follow_the_order_of_requests():
    # each request needs prompt + 7 positions, rounded up to 64
    lengths = [10, 60, 120, 5, 5, 5, 200]
    batches = plan_batches(lengths, 8, max_tokens=256, max_slots=8, sequence_limit=1024)
    assert batches == [[0, 1], [2, 3, 4], [5], [6]]
    for batch in batches:
        assert sum((lengths[i] + 7 + 63) // 64 * 64 for i in batch) <= 256
    assert sum(batches, []) == list(range(7))
    assert plan_batches([5] * 5, 4, 10 ** 6, max_slots=8, sequence_limit=64, batch_size=2) == [[0, 1], [2, 3], [4]]
    assert plan_batches([5] * 5, 4, 10 ** 6, max_slots=2, sequence_limit=64) == [[0, 1], [2, 3], [4]]
    with pytest.raises(bt.GenerationError, match="the limit is 64"):
        plan_batches([60], 6, 10 ** 6, 8, sequence_limit=64)
    assert plan_batches([60], 5, 10 ** 6, 8, sequence_limit=64) == [[0]]       # 60 + 5 - 1 = 64 fits
    with pytest.raises(bt.GenerationError, match="cache holds 128"):
        plan_batches([130], 2, 128, 8, sequence_limit=1024)
    with pytest.raises(bt.GenerationError, match="empty"):
        plan_batches([3, 0], 2, 128, 8, 64)


def test_limits_of_unequal_prompts_that_grow_to_one_total_length():
    assert new_token_limits([5, 60, 63], 100, None) == [100, 100, 100]
    assert new_token_limits([5, 60, 63], 10, total_length=64) == [10, 4, 1]
    with pytest.raises(bt.GenerationError, match="prompt 1 holds 64 tokens already"):
        new_token_limits([5, 64], 10, total_length=64)
    # each request is sized by its own limit: 60 + 4 - 1 and 63 + 1 - 1 positions fit a limit of 64
    assert plan_batches([5, 60, 63], [10, 4, 1], 10 ** 6, 8, sequence_limit=64) == [[0, 1, 2]]
    with pytest.raises(bt.GenerationError, match="prompt 1: 60 prompt tokens \\+ 6 new tokens need 65"):
        plan_batches([5, 60], [10, 6], 10 ** 6, 8, sequence_limit=64)
    config = bt.GenerationConfig(max_new_tokens=5, eos_token_ids=[9])
    tracker = GenerationTracker(config, [3, 3], limits=[2, None])
    assert tracker.push(0, 1, -0.1) is None and tracker.push(0, 2, -0.1).kind == "length"
    assert tracker.push(1, 1, -0.1) is None and tracker.push(1, 2, -0.1) is None
    assert stop_decision(config, [1, 9], limit=2).kind == "eos"          # end-of-sequence still beats length


def test_chunks_cover_every_prompt_once_and_rows_run_out():
    """The reference cuts chunks on columns (src/generation/layout.rs:259-319); rows that have no
    token in a chunk are absent from it."""
    assert prefill_chunks([1, 23], None) == [[(0, 0, 1), (1, 0, 23)]]
    chunks = prefill_chunks([1, 23], 7)
    assert chunks == [[(0, 0, 1), (1, 0, 7)], [(1, 7, 14)], [(1, 14, 21)], [(1, 21, 23)]]
    for lengths, size in (([5, 11, 17], 4), ([64, 3, 65], 64), ([9], 100)):
        covered = {row: [] for row in range(len(lengths))}
        for step in prefill_chunks(lengths, size):
            assert step and all(0 < end - begin <= size for _, begin, end in step)
            for row, begin, end in step:
                covered[row] += list(range(begin, end))
        assert all(covered[row] == list(range(n)) for row, n in enumerate(lengths))
    with pytest.raises(bt.GenerationError, match="greater than zero"):
        prefill_chunks([3], 0)


def test_decoding_one_step_ahead_feeds_the_right_rows_and_drops_what_a_stop_made_useless():
    """The decode loop that keeps the host a step behind the GPU, with a scripted engine and
    sampler (no GPU): every step feeds exactly the rows that can still go on unless their pending
    token stops them; a row that ends by its length is never fed again; a row that its token ends
    was fed once more, its slot is closed and its logits row is dropped before the next
    selection; tokens, order of callbacks and finish reasons are those of the scripted tokens."""
    import torch
    from burn_transformers_amd.engine.generate import _decode_ahead

    # what each row will be given, token by token: row 0 stops at its third token (7 is end-of-sequence),
    # row 1 runs into its own limit of 2, row 2 into max_new_tokens = 5
    script = {0: [3, 4, 7, 9, 9], 1: [5, 6, 9, 9, 9], 2: [1, 2, 3, 4, 5]}
    config = bt.GenerationConfig(max_new_tokens=5, eos_token_ids=[7])
    tracker = GenerationTracker(config, [4, 4, 4], limits=[5, 2, 5])

    class Engine:
        device = torch.device("cpu")

        def __init__(self):
            self.fed, self.closed = [], []

        def step(self, entries, device_tokens=None):
            assert all(tokens == [0] for _, tokens in entries) and device_tokens.numel() == len(entries)
            self.fed.append([slot for slot, _ in entries])
            return torch.tensor([[float(slot)] for slot, _ in entries])     # a "logits" row that names its slot

        def close(self, slot):
            self.closed.append(slot)

    class Sampler:
        def __init__(self):
            self.seen, self.steps = [], {row: 0 for row in script}

        def launch(self, logits, rows):
            assert logits.shape[0] == len(rows)
            self.seen.append((logits[:, 0].tolist(), list(rows)))
            self.rows = list(rows)

        def device_ids(self, count):
            return torch.zeros(count, dtype=torch.int32)

        def result(self):
            ids = [script[row][self.steps[row]] for row in self.rows]
            for row in self.rows:
                self.steps[row] += 1
            return ids, [-0.5] * len(ids)

    engine, sampler = Engine(), Sampler()
    slots = [10, 11, 12]
    open_rows, events = {0, 1, 2}, []
    first = torch.tensor([[10.0], [11.0], [12.0]])
    _decode_ahead(engine, sampler, tracker, slots, open_rows, first, [0, 1, 2],
                  lambda row, token, logp, reason: events.append((row, token, str(reason) if reason else None)))
    assert [s.token_ids for s in tracker.sequences] == [[3, 4, 7], [5, 6], [1, 2, 3, 4, 5]]
    assert [str(s.finish_reason) for s in tracker.sequences] == ["EndOfSequence(token_id=7)", "Length", "Length"]
    # step by step: all three; row 1's second token is its last, so it is not fed; row 0 is fed with
    # the token that ends it (nobody knew), then is gone; row 2's fifth token is its last
    assert engine.fed == [[10, 11, 12], [10, 12], [10, 12], [12]]
    assert engine.closed == [11, 10, 12] and open_rows == set()
    # every selection saw the logits rows of exactly its live rows, in order
    assert sampler.seen == [([10.0, 11.0, 12.0], [0, 1, 2]), ([10.0, 11.0, 12.0], [0, 1, 2]), ([10.0, 12.0], [0, 2]),
                            ([12.0], [2]), ([12.0], [2])]
    assert [e[:2] for e in events] == [(0, 3), (1, 5), (2, 1), (0, 4), (1, 6), (2, 2), (0, 7), (2, 3), (2, 4), (2, 5)]
