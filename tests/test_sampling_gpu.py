"""Selection with processed logits (bias, penalties, banned tokens, top-k / top-p / min-p) against
the plain functions of tests/plain_gpt2.py, then through the generation loop."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from model_helpers import CONFIGS, model_folder, plain_logits, prompts_for  # noqa: E402

DEV = "cuda:0"


def make_rows(rows, vocab, seed, spread=3.0):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, vocab, generator=gen) * spread
    counts_all = (torch.rand(rows + 2, vocab, generator=gen) < 0.05).to(torch.int32) * \
        torch.randint(1, 4, (rows + 2, vocab), generator=gen, dtype=torch.int32)
    counts_gen = torch.minimum(counts_all, (torch.rand(rows + 2, vocab, generator=gen) < 0.5).to(torch.int32) * 5)
    return logits, counts_all, counts_gen


def run_kernel(logits, batch_rows, **kw):
    rows = logits.shape[0]
    ids = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    logp = torch.full((rows,), float("nan"), dtype=torch.float32, device=DEV)
    dev = {k: (v.to(DEV) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    K.select_processed(logits.to(DEV), ids, logp, batch_rows=torch.tensor(batch_rows, dtype=torch.int32, device=DEV), **dev)
    return ids.tolist(), logp.tolist()


@pytest.mark.parametrize("vocab", [517, 50257, 70001])
def test_greedy_after_bias_penalties_and_bans(vocab):
    rows = 6
    logits, counts_all, counts_gen = make_rows(rows, vocab, seed=vocab)
    batch_rows = [5, 0, 7, 2, 3, 1]                     # rows of the batch as it started: where the counts live
    bias = torch.zeros(vocab)
    bias[3], bias[vocab - 1], bias[100] = 4.0, -50.0, 2.5
    banned = [[int(logits[r].argmax())] + [7, 8] if r % 2 == 0 else [] for r in range(rows)]
    offsets = [0]
    for b in banned:
        offsets.append(offsets[-1] + len(b))
    ids, logp = run_kernel(logits, batch_rows, bias=bias, counts_all=counts_all, counts_add=counts_gen,
                           ban_ids=torch.tensor([t for b in banned for t in b], dtype=torch.int32),
                           ban_offsets=torch.tensor(offsets, dtype=torch.int32),
                           repetition=1.7, presence=0.6, frequency=0.3, clamp=True)
    for r in range(rows):
        z = plain.process_logits(logits[r], sampling=False, logit_bias={3: 4.0, vocab - 1: -50.0, 100: 2.5},
                                 repetition_penalty=1.7, presence_penalty=0.6, frequency_penalty=0.3,
                                 seen_counts=counts_all[batch_rows[r]], additive_counts=counts_gen[batch_rows[r]],
                                 banned=banned[r])
        assert ids[r] == int(z.argmax()) and ids[r] not in banned[r]
        assert abs(logp[r] - float(torch.log_softmax(z, -1)[ids[r]])) < 2e-4


CASES = [dict(top_k=1), dict(top_k=5), dict(top_k=50), dict(top_p=0.1), dict(top_p=0.5), dict(top_p=0.9),
         dict(min_p=0.05), dict(min_p=0.5), dict(top_k=40, top_p=0.8), dict(top_k=200, top_p=0.95, min_p=0.02),
         dict(top_p=0.7, min_p=0.3)]


@pytest.mark.parametrize("vocab", [517, 50257])
@pytest.mark.parametrize("case", CASES, ids=[",".join(f"{k}={v}" for k, v in c.items()) for c in CASES])
def test_sampling_from_the_truncated_distribution(vocab, case):
    """The log-probability returned is that of the chosen token among the survivors, so it agrees
    with the plain filters only if the same tokens survived; the choice is the inverse CDF."""
    rows, temperature, seed, first = 12, 0.7, 99, 1000
    logits, counts_all, counts_gen = make_rows(rows, vocab, seed=3, spread=2.0)
    batch_rows = list(range(rows - 1, -1, -1))
    ids, logp = run_kernel(logits, batch_rows, temperature=temperature, clamp=True, seed=seed, first_draw=first, **case)
    checked = 0
    for r in range(rows):
        z = plain.process_logits(logits[r], sampling=True, temperature=temperature)
        kept = plain.truncate(z, **case)
        near_boundary = False
        if "top_p" in case:      # is some item's mass-before within float32 rounding of p?  Then one item may go either way
            ranked = torch.softmax(torch.sort(plain.truncate(z, top_k=case.get("top_k")), descending=True).values, -1)
            before = torch.cumsum(ranked, -1) - ranked
            edge = int((before - case["top_p"]).abs().argmin())
            near_boundary = float((before[edge] - case["top_p"]).abs()) < 1e-5
            if near_boundary and float(ranked[edge]) > 1e-4:
                continue                                 # a heavy item on the fence: its fate changes every number below
        checked += 1
        p = torch.softmax(kept, -1)
        k = ids[r]
        assert float(p[k]) > 0.0 or near_boundary, f"row {r}: token {k} did not survive {case}"
        if float(p[k]) > 0.0:
            assert abs(logp[r] - math.log(float(p[k]))) < 3e-4, (r, case)
            u = plain.interior_unit(plain.splitmix64(seed, first + batch_rows[r]))
            c = torch.cumsum(p, -1)
            lo = float(c[k - 1]) if k > 0 else 0.0
            assert lo - 1e-4 <= u <= float(c[k]) + 1e-4, (r, k, u)
    assert checked >= rows - 2


def test_cutting_off_is_refused_beyond_what_a_work_group_holds():
    logits = torch.zeros(2, 70001)
    with pytest.raises(K.KernelError, match="outside 1..65536"):
        run_kernel(logits, [0, 1], temperature=1.0, top_k=5)
    ids, logp = run_kernel(logits, [0, 1], temperature=1.0, repetition=1.3,
                           counts_all=torch.ones(2, 70001, dtype=torch.int32))      # nothing cut off: any size
    assert all(0 <= i < 70001 for i in ids)


def test_rows_where_everything_is_tied_or_banned():
    vocab = 300
    logits = torch.zeros(3, vocab)
    logits[1, 17] = 1.0
    ban = list(range(vocab))
    ids, logp = run_kernel(logits, [0, 1, 2], temperature=1.0, top_k=3, top_p=0.5, seed=1,
                           ban_ids=torch.tensor(ban, dtype=torch.int32),
                           ban_offsets=torch.tensor([0, 0, 0, vocab], dtype=torch.int32))
    # row 0: all scores tied, so top-k keeps all of them (ties with the boundary survive) and the nucleus
    # keeps every token tied with its last member: a uniform draw over the vocabulary
    assert 0 <= ids[0] < vocab and abs(logp[0] - math.log(1.0 / vocab)) < 1e-4
    # row 1: three survive top-k?  No: the boundary (third greatest) is the tied zero, so all survive it; the
    # nucleus of 0.5 then needs the single larger token and the zeros tied at its edge
    assert 0 <= ids[1] < vocab
    # row 2: every token banned: nothing can be chosen, and the log-probability says so
    assert ids[2] == 0 and logp[2] == -math.inf


def test_generation_with_penalties_follows_the_plain_loop():
    """Greedy generation in float32 with bias, repetition, presence and frequency penalties, banned
    n-grams and end-of-sequence held back, against the same loop over the plain model's logits."""
    name = "A"
    folder, cfg, weights = model_folder(name)
    model = bt.load_model(folder, dtype="float32")
    engine = bt.Engine(model, max_tokens=1024)
    prompts = prompts_for(name, [9, 30, 17], seed=21)
    first = int(plain_logits(name, prompts[0])[-1].argmax())
    config = bt.GenerationConfig(max_new_tokens=14, min_new_tokens=6, eos_token_ids=[first], repetition_penalty=1.4,
                                 presence_penalty=0.3, frequency_penalty=0.2, no_repeat_ngram_size=2,
                                 logit_bias={5: 1.5, 6: -2.0}, additive_penalty_scope="generated")
    got = bt.generate(engine, prompts, config)
    vocab = cfg["vocab_size"]
    for prompt, sequence in zip(prompts, got):
        tokens, emitted = list(prompt), []
        while True:
            z = plain_logits(name, tokens)[-1]
            seen = torch.bincount(torch.tensor(tokens), minlength=vocab)
            generated = torch.bincount(torch.tensor(emitted, dtype=torch.int64), minlength=vocab)
            banned = plain.banned_by_ngrams(tokens, 2) + ([first] if len(emitted) < 6 else [])
            z = plain.process_logits(z, sampling=False, logit_bias={5: 1.5, 6: -2.0}, repetition_penalty=1.4,
                                     presence_penalty=0.3, frequency_penalty=0.2, seen_counts=seen,
                                     additive_counts=generated, banned=banned)
            token = int(z.argmax())
            tokens.append(token)
            emitted.append(token)
            if (token == first and len(emitted) >= 6) or len(emitted) == 14:
                break
        assert sequence.token_ids == emitted
        assert first not in emitted[:6]
        for i in range(len(prompt), len(tokens)):       # no generated token completes a bigram seen before it
            assert (tokens[i - 1], tokens[i]) not in set(zip(tokens[:i - 1], tokens[1:i]))


def test_sampled_generation_with_truncation_is_reproducible_and_respects_top_k():
    folder, cfg, _ = model_folder("BW")
    model = bt.load_model(folder, dtype="bfloat16")
    engine = bt.Engine(model, max_tokens=1024)
    prompts = prompts_for("BW", [5, 40], seed=2)
    config = bt.GenerationConfig(max_new_tokens=12, strategy="sample", temperature=0.9, top_k=1, top_p=0.9, seed=4)
    sampled = bt.generate(engine, prompts, config)
    greedy = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=12))
    assert [s.token_ids for s in sampled] == [g.token_ids for g in greedy]      # top_k = 1 leaves the maximum only
    assert all(abs(lp) < 1e-5 for s in sampled for lp in s.log_probabilities)   # which then has probability one
    config = bt.GenerationConfig(max_new_tokens=12, strategy="sample", temperature=1.3, top_k=20, top_p=0.95, min_p=0.01,
                                 repetition_penalty=1.1, seed=11)
    once, again = bt.generate(engine, prompts, config), bt.generate(engine, prompts, config)
    assert [s.token_ids for s in once] == [s.token_ids for s in again]
    other = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=12, strategy="sample", temperature=1.3,
                                                             top_k=20, top_p=0.95, min_p=0.01, repetition_penalty=1.1, seed=12))
    assert [s.token_ids for s in once] != [s.token_ids for s in other]


def test_a_row_keeps_the_draws_of_its_place_in_the_batch_as_it_started():
    """Three rows start together; the middle one ends after its first token.  The reference keeps
    the finished row in the batch and reserves a draw for it in every selection
    (src/generation.rs:667-699: one block of ``batch`` counters per call), so the third row goes on
    with draws s * 3 + 2.  Had the draws been numbered by the rows still alive it would use
    s * 2 + 1: in every step where the two candidate draws choose different tokens from the plain
    implementation's distribution, the generated token is the first candidate's."""
    name, seed = "A", 5
    folder, config, weights = model_folder(name, 8.0)
    model = bt.load_model(folder, dtype="float32", device=DEV)
    engine = bt.Engine(model, max_tokens=1024)
    prompts = prompts_for(name, [9, 30, 17], seed=61)
    steps = 24
    cfg = bt.GenerationConfig(max_new_tokens=steps, strategy="sample", temperature=1.0, seed=seed)
    # the middle row may hold 31 tokens in all: it ends, by its length, with its first new token
    out = bt.generate(engine, prompts, cfg, total_length=31)
    assert [len(s.token_ids) for s in out] == [22, 1, 14]
    separated = 0
    for row, alive_index in ((0, 0), (2, 1)):
        sequence = out[row]
        logits = plain.forward(prompts[row] + sequence.token_ids, weights, config)
        for s, token in enumerate(sequence.token_ids):
            z = logits[len(prompts[row]) - 1 + s]
            c = torch.cumsum(torch.softmax(z, -1), -1)
            as_started = plain.interior_unit(plain.splitmix64(seed, s * 3 + row))
            low = float(c[token - 1]) if token else 0.0
            assert low - 1e-5 <= as_started <= float(c[token]) + 1e-5, f"row {row} step {s}"
            if s == 0 or row == 0:
                continue
            by_alive_rows = plain.interior_unit(plain.splitmix64(seed, s * 2 + alive_index))
            other = plain.sample_index(z, 1.0, by_alive_rows)
            edge = min(abs(by_alive_rows - low), abs(by_alive_rows - float(c[token])))
            if other != token and edge > 1e-4:
                separated += 1
    assert separated >= 8, f"only {separated} steps tell the two numberings apart"


def test_the_log_probability_of_a_sampled_token_is_that_of_the_tempered_distribution():
    """Logits ln 1, ln 2, ln 3, ln 4 (then nothing: -inf would be a probability of 0 as well, here the
    vocabulary simply ends) at temperature 0.5 are probabilities 1, 4, 9, 16 over 30, so the chosen
    token's log-probability is ln(k^2 / 30) where the raw distribution would give ln(k / 10): the
    two differ by ln(k / 3), worked by hand, and greedy selection reports the raw one
    (src/generation.rs:732-743: the log-softmax of the PROCESSED logits, and temperature is part of
    the processing only when sampling, :35-37)."""
    vocab = 4
    rows = 64
    z = torch.log(torch.arange(1, vocab + 1, dtype=torch.float32)).repeat(rows, 1).to(DEV)
    config = bt.GenerationConfig(max_new_tokens=1, strategy="sample", temperature=0.5, seed=123)
    sampler = bt.Sampler(config, rows, torch.device(DEV), vocab)
    ids, logps = sampler.select(z, list(range(rows)))
    edges = [0.0, 1 / 30, 5 / 30, 14 / 30, 1.0]
    chosen = set()
    for row, (token, logp) in enumerate(zip(ids, logps)):
        u = plain.interior_unit(plain.splitmix64(123, row))
        assert edges[token] - 1e-6 <= u <= edges[token + 1] + 1e-6, f"row {row}"
        k = token + 1
        assert abs(logp - math.log(k * k / 30)) < 1e-5
        assert abs((logp - math.log(k / 10)) - math.log(k / 3)) < 1e-5      # tempered minus raw, by hand
        chosen.add(token)
    assert len(chosen) >= 3            # the draws reach most tokens, so every k above was exercised
    greedy = bt.Sampler(bt.GenerationConfig(max_new_tokens=1, temperature=0.5), rows, torch.device(DEV), vocab)
    ids, logps = greedy.select(z, list(range(rows)))
    assert set(ids) == {3} and all(abs(logp - math.log(4 / 10)) < 1e-5 for logp in logps)
