"""Typed configuration and the registry (no GPU)."""

import json

import pytest

import burn_transformers_amd as bt
from burn_transformers_amd.config.gpt2 import GPT2Config


def test_defaults_are_gpt2_small():
    """src/models/gpt2.rs:149-171."""
    c = GPT2Config.from_dict({})
    assert (c.vocab_size, c.n_embd, c.n_layer, c.n_head, c.n_positions) == (50257, 768, 12, 12, 1024)
    assert c.n_inner is None and c.intermediate_size == 3072 and c.head_size == 64
    assert c.activation_function == "gelu_new" and c.layer_norm_epsilon == 1e-5
    assert c.scale_attn_weights and not c.scale_attn_by_inverse_layer_idx and c.tie_word_embeddings


def test_aliases_unknown_keys_and_wrappers():
    c = GPT2Config.from_dict({"hidden_size": 96, "num_hidden_layers": 3, "num_attention_heads": 2,
                              "max_position_embeddings": 64, "resid_pdrop": 0.1, "unknown_key": [1, 2]})
    assert (c.n_embd, c.n_layer, c.n_head, c.n_positions) == (96, 3, 2, 64)
    wrapped = GPT2Config.from_dict({"text_config": {"n_embd": 32, "n_head": 2}, "model_type": "gpt2"})
    assert wrapped.n_embd == 32
    assert GPT2Config.from_dict({"n_inner": None}).intermediate_size == 4 * 768
    assert GPT2Config.from_dict({"n_inner": 320, "n_embd": 96, "n_head": 2}).intermediate_size == 320


@pytest.mark.parametrize("patch,field", [
    ({"model_type": "llama"}, "model_type"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"vocab_size": 0, "n_embd": 0}, "vocab_size"),          # the first bad extent is the one named
    ({"n_embd": 2 ** 31}, "n_embd"),
    ({"n_layer": 0}, "n_layer"),
    ({"n_layer": 2 ** 18 + 1}, "n_layer"),
    ({"n_head": 5}, "n_head"),
    ({"n_positions": -3}, "n_positions"),
    ({"layer_norm_epsilon": 0.0}, "layer_norm_epsilon"),
    ({"layer_norm_epsilon": float("nan")}, "layer_norm_epsilon"),
    ({"initializer_range": -1.0}, "initializer_range"),
    ({"reorder_and_upcast_attn": True}, "reorder_and_upcast_attn"),
    ({"add_cross_attention": True}, "add_cross_attention"),
    ({"tie_word_embeddings": False}, "tie_word_embeddings"),
    ({"causal": False}, "causal"),
    ({"n_inner": 0}, "n_inner"),
    ({"activation_function": "relu"}, "activation_function"),
    ({"n_embd": "wide"}, "n_embd"),
    ({"scale_attn_weights": 1}, "scale_attn_weights"),
])
def test_each_bad_field_is_named(patch, field):
    """src/models/gpt2_tests.rs:26-82: the message is `gpt2.<field>: reason`."""
    with pytest.raises(bt.ConfigError) as info:
        GPT2Config.from_dict(patch)
    assert info.value.field == field and str(info.value).startswith(f"gpt2.{field}: ")


def test_head_count_message():
    with pytest.raises(bt.ConfigError, match=r"gpt2\.n_head: must divide n_embd"):
        GPT2Config.from_dict({"n_embd": 100, "n_head": 3})


def test_registry_resolves_architectures_first_then_model_type():
    family = bt.resolve_family({"architectures": ["GPT2LMHeadModel"]})
    assert family.name == "gpt2" and family is bt.resolve_family({"model_type": "gpt2"})
    assert family is bt.resolve_family({"architectures": ["SomethingElse"], "model_type": "gpt2"})
    with pytest.raises(bt.UnsupportedArchitecture, match="`LlamaForCausalLM`.*supported values: GPT2LMHeadModel, gpt2"):
        bt.resolve_family({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(bt.UnsupportedArchitecture, match="nothing"):
        bt.resolve_family({})


def test_registering_another_family():
    toy = bt.Family(name="toy", architectures=("ToyLM",), model_types=("toy",), config_class=GPT2Config,
                    plan=lambda c: None, contract=lambda c: None, init=lambda c, g: {})
    bt.register_family(toy)
    try:
        assert bt.resolve_family({"architectures": ["ToyLM"]}) is toy
        clash = bt.Family(name="other", architectures=("ToyLM",), model_types=(), config_class=GPT2Config,
                          plan=None, contract=None, init=None)
        with pytest.raises(ValueError, match="already registered"):
            bt.register_family(clash)
    finally:
        bt.unregister_family("toy")
    assert "ToyLM" not in bt.supported_names()


def test_plan_is_data_taken_from_the_configuration():
    c = GPT2Config.from_dict({"n_layer": 3, "n_embd": 96, "n_head": 2, "n_inner": 320, "vocab_size": 517,
                              "n_positions": 64, "activation_function": "gelu", "layer_norm_epsilon": 1e-6,
                              "scale_attn_by_inverse_layer_idx": True})
    plan = bt.resolve_family({"model_type": "gpt2"}).plan(c)
    assert (plan.width, plan.vocab_size, plan.max_positions, len(plan.layers)) == (96, 517, 64, 3)
    assert [(e.layer, e.cache, e.writes) for e in plan.schedule] == [(0, 0, True), (1, 1, True), (2, 2, True)]
    mixer = plan.layers[2].parts["mixer"]
    assert mixer.kind == "attention" and mixer.params["head_dim"] == 48 and mixer.params["kv_heads"] == 2
    assert mixer.params["scale"] == pytest.approx(1 / (48 ** 0.5) / 3)      # layer index 2 -> divide by 3
    ff = plan.layers[0].parts["ff"]
    assert ff.params == {"width": 96, "inner": 320, "activation": "gelu_erf"}
    assert plan.layers[1].parts["ff_norm"].params["eps"] == 1e-6
    assert plan.readout.tensors["weight"] == plan.embedding.tensors["tokens"] == "wte.weight"
    assert json.dumps(c.to_dict())      # what random-weights mode writes as config.json
