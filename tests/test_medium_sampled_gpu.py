"""GPT-2 medium's sizes, 64 unequal prompts prefilled in chunks of 256, then sampled at temperature 1.

24 layers of width 1,024, 16 heads of 64, inner width 4,096, 50,257 tokens, 1,024 positions, random
weights, in float32 and in bfloat16: 64 prompts of 64 to 768 tokens (the ends of the range and the
chunk's edges made sure of) go through ``generate`` with ``prefill_chunk=256`` as ONE batch (so the
later chunks hold fewer and fewer rows, each from the chunk in which its prompt ends), then 12
tokens each are sampled at temperature 1.0.  For six requests every sampled token is checked
against the plain implementation: it is the inverse-CDF choice of its draw (number ``step * 64 +
row`` of the seed's stream) on softmax(z), and its log-probability is log_softmax(z)[token].  In
float32 the prompts fed whole give the same tokens and log-probabilities as in chunks (the
reference asks the same of its loop: src/generation/causal_tests.rs:524-576)."""

import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.slow]

import burn_transformers_amd as bt  # noqa: E402
import plain_gpt2 as plain  # noqa: E402

MEDIUM = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 24, "n_embd": 1024, "n_head": 16,
          "n_inner": 4096, "vocab_size": 50257, "n_positions": 1024, "activation_function": "gelu_new",
          "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
BATCH, CHUNK, NEW_TOKENS, SEED = 64, 256, 12, 29
CHECKED = [0, 1, 2, 3, 4, 40]          # rows whose lengths are 64, 768, 256, 257, 512 and a drawn one
_held = {}


def medium():
    if not _held:
        print("[medium] drawing 3.5e8 weights", flush=True)
        _, tensors = bt.random_tensors(MEDIUM, 17)
        # the token table three times as large: logits with a spread of some units, so that a draw
        # falls on a token whose probability stands well above the float32 rounding of the sums
        tensors["wte.weight"] = tensors["wte.weight"] * 3.0
        tensors = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v.float()) for k, v in tensors.items()}
        gen = torch.Generator().manual_seed(23)
        lengths = torch.randint(64, 769, (BATCH,), generator=gen).tolist()
        lengths[:5] = [64, 768, 256, 257, 512]
        prompts = [torch.randint(0, MEDIUM["vocab_size"], (n,), generator=gen).tolist() for n in lengths]
        _held.update(tensors=tensors, wide={k: v.double() for k, v in tensors.items()}, prompts=prompts, oracle={})
    return _held


def oracle(row, tokens):
    """float64 logits of the plain implementation at the places the sampled tokens were chosen from."""
    held = medium()
    key = (row, tuple(tokens))
    if key not in held["oracle"]:
        prompt = held["prompts"][row]
        print(f"[medium] plain forward of {len(prompt)} + {len(tokens)} tokens through 24 layers", flush=True)
        rows = list(range(len(prompt) - 1, len(prompt) - 1 + len(tokens)))
        held["oracle"][key] = plain.forward(prompt + list(tokens[:-1]), held["wide"], MEDIUM, rows=rows)
    return held["oracle"][key]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_64_unequal_prompts_in_chunks_of_256_then_sampled_at_temperature_1(dtype):
    held = medium()
    prompts = held["prompts"]
    model = bt.model_from_tensors(MEDIUM, held["tensors"], dtype=dtype, device="cuda:0")
    budget = sum((len(p) + NEW_TOKENS + 63) // 64 * 64 for p in prompts)
    engine = bt.Engine(model, max_tokens=budget)
    config = bt.GenerationConfig(max_new_tokens=NEW_TOKENS, strategy="sample", temperature=1.0, seed=SEED)
    chunked = bt.generate(engine, prompts, config, prefill_chunk=CHUNK, total_length=MEDIUM["n_positions"])
    engine.cache.ledger.check()
    assert engine.cache.ledger.live_slots() == []
    assert all(len(s.token_ids) == NEW_TOKENS and str(s.finish_reason) == "Length" for s in chunked)
    # the distributions are neither uniform nor one-hot: a draw decides, and it can be checked
    band = 5e-5 if dtype == "float32" else 3e-2
    for row in CHECKED:
        sequence = chunked[row]
        logits = oracle(row, sequence.token_ids) if dtype == "float32" else \
            plain.forward(prompts[row] + sequence.token_ids[:-1], held["wide"], MEDIUM,
                          rows=list(range(len(prompts[row]) - 1, len(prompts[row]) - 1 + NEW_TOKENS)))
        worst = 0.0
        for s, (token, logp) in enumerate(zip(sequence.token_ids, sequence.log_probabilities)):
            u = plain.interior_unit(plain.splitmix64(SEED, s * BATCH + row))
            z = logits[s]
            c = torch.cumsum(torch.softmax(z, -1), -1)
            low = float(c[token - 1]) if token else 0.0
            assert low - band <= u <= float(c[token]) + band, \
                f"row {row} ({len(prompts[row])} prompt tokens) step {s}: token {token} covers " \
                f"({low}, {float(c[token])}], the draw is {u}"
            if dtype == "float32":
                assert token == plain.sample_index(z, 1.0, u) or min(u - low, float(c[token]) - u) < band
            error = abs(logp - plain.log_probability(z, token, 1.0))
            worst = max(worst, error)
            assert error < (1e-4 if dtype == "float32" else 6e-2), f"row {row} step {s}: log-probability off by {error}"
        print(f"[medium] {dtype} row {row}: {len(prompts[row])} prompt tokens, log-probabilities within {worst:.3g}", flush=True)
    if dtype == "float32":
        whole = bt.generate(engine, prompts, config, total_length=MEDIUM["n_positions"])
        differing = [i for i in range(BATCH) if whole[i].token_ids != chunked[i].token_ids]
        assert not differing, f"rows {differing} got other tokens from whole prompts than from chunks"
        gap = max(abs(a - b) for w, c in zip(whole, chunked) for a, b in zip(w.log_probabilities, c.log_probabilities))
        assert gap < 1e-4, f"log-probabilities of whole and chunked prompts differ by {gap}"
