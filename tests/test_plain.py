"""Pins of the plain implementation: what fixes each formula beside the reference's text."""

import json
import math
import os

import pytest
import torch

import plain_gpt2 as plain

FIXTURE = os.path.join(os.path.dirname(__file__), "fixtures", "gpt2_tiny_reference.json")


def fixture_weights(shapes):
    """The reference's xorshift64 generator (src/models/gpt2/prepare_reference.py:19-38,
    src/models/gpt2/model_tests.rs:50-86): tensors in sorted-name order."""
    mask = (1 << 64) - 1
    weights = {}
    for index, name in enumerate(sorted(shapes)):
        shape = shapes[name]
        state = (20260910 ^ ((index + 1) * 0x9E3779B97F4A7C15)) & mask
        is_scale = name.endswith(".weight") and (".ln_" in name or name.startswith("ln_f."))
        shift = 32 if name.endswith(".bias") else 23 if name.endswith("mlp.c_fc.weight") else 29
        values = []
        for _ in range(math.prod(shape)):
            state ^= (state << 13) & mask
            state ^= state >> 7
            state ^= (state << 17) & mask
            value = ((state >> 40) - (1 << 23)) / (1 << shift)
            values.append(1.0 + value if is_scale else value)
        weights[name] = torch.tensor(values, dtype=torch.float32).reshape(shape)
    return weights


@pytest.fixture(scope="module")
def reference():
    with open(FIXTURE) as handle:
        return json.load(handle)


@pytest.mark.parametrize("activation", ["gelu_new", "gelu"])
def test_reference_vector(reference, activation):
    """The reference's own PyTorch vector (fixtures/tiny_reference.json; tolerances of
    src/models/gpt2/model_tests.rs:189,196,202).  Fixes Conv1D orientation, q/k/v order,
    pre-norm placement, both GELUs, the tied readout and causal masking."""
    weights = fixture_weights(reference["parameter_shapes"])
    cfg = dict(reference["config"], activation_function=activation)
    expected = reference["references"][activation]
    for row, (ids, mask) in enumerate(zip(reference["input_ids"], reference["token_mask"])):
        length = sum(mask)
        assert mask == [1] * length + [0] * (len(mask) - length)
        taps = {}
        logits = plain.forward(ids[:length], weights, cfg, torch.float32, taps)
        want = torch.tensor(expected["logits"][row])[:length]
        assert (logits - want).abs().max() <= 2e-6
        hidden = expected["hidden_states"]
        assert (taps["hidden"][0] - torch.tensor(hidden[0][row])[:length]).abs().max() <= 3e-6
        assert (taps["hidden"][1] - torch.tensor(hidden[1][row])[:length]).abs().max() <= 3e-6
        assert (taps["final"] - torch.tensor(hidden[2][row])[:length]).abs().max() <= 3e-6
        for layer in range(cfg["n_layer"]):
            want = torch.tensor(expected["mlp_outputs"][f"mlp_{layer}"][row])[:length]
            assert (taps["mlp"][layer] - want).abs().max() <= 2e-6


def test_fixture_separates_the_two_gelus(reference):
    """src/models/gpt2/model_tests.rs:158-164."""
    a = torch.tensor(reference["references"]["gelu"]["logits"])
    b = torch.tensor(reference["references"]["gelu_new"]["logits"])
    assert (a - b).abs().max() > 1e-5
    weights = fixture_weights(reference["parameter_shapes"])
    ids = reference["input_ids"][0]
    x = plain.forward(ids, weights, dict(reference["config"], activation_function="gelu"))
    y = plain.forward(ids, weights, dict(reference["config"], activation_function="gelu_new"))
    assert (x - y).abs().max() > 1e-5


def test_layer_norm_reduces_to_library_and_invariants():
    torch.manual_seed(0)
    x = torch.randn(5, 37, dtype=torch.float64) * 3 + 1.5
    gamma = torch.randn(37, dtype=torch.float64)
    beta = torch.randn(37, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (37,), gamma, beta, 1e-3)
    assert (plain.layer_norm(x, gamma, beta, 1e-3) - want).abs().max() < 1e-12
    ones, zeros = torch.ones(37, dtype=torch.float64), torch.zeros(37, dtype=torch.float64)
    y = plain.layer_norm(x, ones, zeros, 1e-12)
    assert y.mean(-1).abs().max() < 1e-12
    assert (y.var(-1, unbiased=False) - 1).abs().max() < 1e-9
    shifted = plain.layer_norm(x + 7.25, gamma, beta, 1e-3)
    assert (shifted - want).abs().max() < 1e-10


def test_gelus_reduce_to_library_routines():
    x = torch.linspace(-6, 6, 241, dtype=torch.float64)
    assert (plain.gelu_erf(x) - torch.nn.functional.gelu(x)).abs().max() < 1e-14
    assert (plain.gelu_tanh(x) - torch.nn.functional.gelu(x, approximate="tanh")).abs().max() < 1e-14
    for value in (-2.0, -0.5, 0.3, 1.7):
        exact = value * (1 + math.erf(value / math.sqrt(2))) / 2
        assert abs(float(plain.gelu_erf(torch.tensor(value, dtype=torch.float64))) - exact) < 1e-15
    assert (plain.gelu_erf(x) - plain.gelu_tanh(x)).abs().max() > 1e-4


def test_attention_reduces_to_plain_softmax_without_mask():
    torch.manual_seed(1)
    q = torch.randn(1, 6, 8, dtype=torch.float64)
    k = torch.randn(1, 6, 8, dtype=torch.float64)
    v = torch.randn(1, 6, 8, dtype=torch.float64)
    want = torch.softmax(q[0] @ k[0].t() * 0.3, dim=-1) @ v[0]
    assert (plain.attention(q, k, v, 0.3, causal=False)[0] - want).abs().max() < 1e-14
    lib = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.3)
    assert (plain.attention(q, k, v, 0.3) - lib).abs().max() < 1e-13


def test_attention_is_causal_bottom_right_and_windowed():
    torch.manual_seed(2)
    q = torch.randn(2, 3, 4, dtype=torch.float64)
    k = torch.randn(2, 7, 4, dtype=torch.float64)
    v = torch.randn(2, 7, 4, dtype=torch.float64)
    base = plain.attention(q, k, v, 0.5)
    # query row i sits at key position i + 4: row 0 must ignore keys 5 and 6
    k2, v2 = k.clone(), v.clone()
    k2[:, 5:] += 10.0
    v2[:, 5:] -= 3.0
    assert torch.equal(plain.attention(q, k2, v2, 0.5)[:, 0], base[:, 0])
    assert not torch.allclose(plain.attention(q, k2, v2, 0.5)[:, 1], base[:, 1])
    # a window of 2 sees exactly the query's own key and the one before it
    k3, v3 = k.clone(), v.clone()
    k3[:, :3] += 5.0
    v3[:, :3] += 5.0
    w = plain.attention(q, k, v, 0.5, window=2)
    assert torch.equal(plain.attention(q, k3, v3, 0.5, window=2)[:, 0], w[:, 0])
    one = plain.attention(q, k, v, 0.5, window=1)
    assert (one - v[:, 4:7]).abs().max() < 1e-14


def tiny(seed=0, layers=2, width=24, heads=3, inner=40, vocab=31, positions=20, **extra):
    gen = torch.Generator().manual_seed(seed)
    cfg = dict(n_layer=layers, n_embd=width, n_head=heads, n_inner=inner, vocab_size=vocab,
               n_positions=positions, layer_norm_epsilon=1e-5, activation_function="gelu_new")
    cfg.update(extra)

    def rnd(*shape, scale=0.2):
        return torch.randn(*shape, generator=gen, dtype=torch.float64) * scale

    w = {"wte.weight": rnd(vocab, width), "wpe.weight": rnd(positions, width),
         "ln_f.weight": 1 + rnd(width), "ln_f.bias": rnd(width)}
    for i in range(layers):
        p = f"h.{i}."
        w.update({p + "ln_1.weight": 1 + rnd(width), p + "ln_1.bias": rnd(width),
                  p + "ln_2.weight": 1 + rnd(width), p + "ln_2.bias": rnd(width),
                  p + "attn.c_attn.weight": rnd(width, 3 * width), p + "attn.c_attn.bias": rnd(3 * width),
                  p + "attn.c_proj.weight": rnd(width, width), p + "attn.c_proj.bias": rnd(width),
                  p + "mlp.c_fc.weight": rnd(width, inner), p + "mlp.c_fc.bias": rnd(inner),
                  p + "mlp.c_proj.weight": rnd(inner, width), p + "mlp.c_proj.bias": rnd(width)})
    return cfg, w


def test_future_tokens_do_not_change_earlier_logits():
    cfg, w = tiny()
    a = plain.forward([3, 1, 4, 1, 5, 9, 2, 6], w, cfg)
    b = plain.forward([3, 1, 4, 1, 5, 30, 29, 28], w, cfg)
    assert torch.equal(a[:5], b[:5])
    assert not torch.allclose(a[5:], b[5:])


def test_inverse_layer_scale_is_undone_by_scaling_queries():
    """Scaling W_q, b_q of layer i by c = i+1 undoes scale_attn_by_inverse_layer_idx
    (src/models/gpt2/model_tests.rs:1346-1387); an off-by-one in i+1 fails this."""
    cfg, w = tiny(seed=3)
    scaled_cfg = dict(cfg, scale_attn_by_inverse_layer_idx=True)
    ids = [7, 8, 9, 10, 11, 12]
    base = plain.forward(ids, w, cfg)
    assert not torch.allclose(plain.forward(ids, w, scaled_cfg), base)
    w2 = dict(w)
    width = cfg["n_embd"]
    for i in range(cfg["n_layer"]):
        p = f"h.{i}.attn.c_attn."
        weight, bias = w[p + "weight"].clone(), w[p + "bias"].clone()
        weight[:, :width] *= (i + 1)
        bias[:width] *= (i + 1)
        w2[p + "weight"], w2[p + "bias"] = weight, bias
    assert (plain.forward(ids, w2, scaled_cfg) - base).abs().max() < 1e-12


def test_permuting_heads_consistently_changes_nothing():
    cfg, w = tiny(seed=4)
    width, heads = cfg["n_embd"], cfg["n_head"]
    size = width // heads
    perm = torch.cat([torch.arange(size) + h * size for h in (2, 0, 1)])
    ids = [1, 2, 3, 4, 5]
    base = plain.forward(ids, w, cfg)
    w2 = dict(w)
    for i in range(cfg["n_layer"]):
        p = f"h.{i}.attn."
        cols = torch.cat([perm, perm + width, perm + 2 * width])
        w2[p + "c_attn.weight"] = w[p + "c_attn.weight"][:, cols]
        w2[p + "c_attn.bias"] = w[p + "c_attn.bias"][cols]
        w2[p + "c_proj.weight"] = w[p + "c_proj.weight"][perm, :]
    assert (plain.forward(ids, w2, cfg) - base).abs().max() < 1e-12


def test_fused_projection_equals_three_projections():
    cfg, w = tiny(seed=5)
    x = torch.randn(4, cfg["n_embd"], dtype=torch.float64)
    width = cfg["n_embd"]
    weight, bias = w["h.0.attn.c_attn.weight"], w["h.0.attn.c_attn.bias"]
    q, k, v = plain.split_qkv(plain.linear(x, weight, bias), width)
    for part, lo in ((q, 0), (k, width), (v, 2 * width)):
        assert torch.allclose(part, x @ weight[:, lo:lo + width] + bias[lo:lo + width], atol=1e-14)


def test_splitmix64_reference_vector_and_uniform_endpoints():
    """src/generation/random_tests.rs:24-43 and :47-49."""
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423,
            4593380528125082431, 16408922859458223821]
    assert [plain.splitmix64(1234567, i) for i in range(5)] == want
    assert plain.interior_unit(0) == 2.0 ** -24
    assert plain.interior_unit((1 << 64) - 1) == 1.0 - 2.0 ** -24


def test_sample_index_is_the_inverse_cdf():
    logits = torch.tensor([0.0, math.log(2.0), math.log(1.0)], dtype=torch.float64)  # p = .25 .5 .25
    assert plain.sample_index(logits, 1.0, 0.1) == 0
    assert plain.sample_index(logits, 1.0, 0.3) == 1
    assert plain.sample_index(logits, 1.0, 0.74) == 1
    assert plain.sample_index(logits, 1.0, 0.76) == 2
    # temperature divides the logits before the softmax: T = 0.5 squares the odds (1:4:1)
    assert plain.sample_index(logits, 0.5, 0.16) == 0
    assert plain.sample_index(logits, 0.5, 0.17) == 1
    assert abs(plain.log_probability(logits, 1) - math.log(0.5)) < 1e-12
    assert abs(plain.log_probability(logits, 1, 0.5) - math.log(4 / 6)) < 1e-12
