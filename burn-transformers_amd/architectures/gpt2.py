"""GPT-2 as a family: its plan, its checkpoint contract and its random initialisation.

This is the only file that knows GPT-2's wiring and tensor names.
  plan      pre-norm blocks of (LayerNorm, full causal multi-head attention with a fused QKV
            projection, LayerNorm, dense GELU feed-forward), learned absolute positions added
            at the embedding, final LayerNorm, readout tied to the token table
            (src/models/gpt2/model.rs:112-165, 218-270, 385-420, 500-513)
  contract  names, shapes and Conv1D [in, out] layout (src/models/gpt2/checkpoint.rs:103-189)
  init      N(0, s^2) tables and projections, s / sqrt(2 L) for the two projections that write
            into the residual stream (src/models/gpt2.rs:219-255); biases, LayerNorm scales and
            shifts are drawn around their usual values with the same s rather than set to 0 / 1,
            so that tests see them (the reference's own fixture generator does the same,
            src/models/gpt2/prepare_reference.py:26-36)
"""

import math

import torch

from ..config.gpt2 import GPT2Config
from ..config.registry import Family, register_family
from ..engine.plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..weights.contract import Contract, TensorSpec

ACTIVATION_KERNEL = {"gelu_new": "gelu_tanh", "gelu": "gelu_erf"}


def attention_scale(config, layer):
    """(1/sqrt(h) if scale_attn_weights) / (layer + 1 if scale_attn_by_inverse_layer_idx), layer
    zero-based, evaluated in float64 (src/models/gpt2/model.rs:121-133)."""
    scale = 1.0 / math.sqrt(config.head_size) if config.scale_attn_weights else 1.0
    if config.scale_attn_by_inverse_layer_idx:
        scale /= float(layer + 1)
    return scale


def plan(config: GPT2Config) -> ModelPlan:
    width, inner, eps = config.n_embd, config.intermediate_size, config.layer_norm_epsilon

    def norm(prefix):
        return PartSpec("layer_norm", {"width": width, "eps": eps},
                        {"weight": prefix + ".weight", "bias": prefix + ".bias"})

    layers = []
    for i in range(config.n_layer):
        p = f"h.{i}."
        mixer = PartSpec("attention", {
            "width": width, "heads": config.n_head, "kv_heads": config.n_head,
            "head_dim": config.head_size, "scale": attention_scale(config, i),
            "causal": config.causal, "window": 0},
            {"qkv_weight": p + "attn.c_attn.weight", "qkv_bias": p + "attn.c_attn.bias",
             "out_weight": p + "attn.c_proj.weight", "out_bias": p + "attn.c_proj.bias"})
        feed_forward = PartSpec("dense", {
            "width": width, "inner": inner,
            "activation": ACTIVATION_KERNEL[config.activation_function]},
            {"up_weight": p + "mlp.c_fc.weight", "up_bias": p + "mlp.c_fc.bias",
             "down_weight": p + "mlp.c_proj.weight", "down_bias": p + "mlp.c_proj.bias"})
        layers.append(LayerPlan("pre_norm", {"mixer_norm": norm(p + "ln_1"), "mixer": mixer,
                                             "ff_norm": norm(p + "ln_2"), "ff": feed_forward}))
    return ModelPlan(
        width=width, vocab_size=config.vocab_size, max_positions=config.n_positions,
        embedding=PartSpec("learned_positions", {"width": width, "vocab_size": config.vocab_size,
                                                 "max_positions": config.n_positions},
                           {"tokens": "wte.weight", "positions": "wpe.weight"}),
        layers=layers,
        schedule=[ScheduleEntry(layer=i, cache=i) for i in range(config.n_layer)],
        final_norm=norm("ln_f"),
        readout=PartSpec("linear_readout", {"width": width, "vocab_size": config.vocab_size},
                         {"weight": "wte.weight"}))


def contract(config: GPT2Config) -> Contract:
    d, m = config.n_embd, config.intermediate_size
    tensors = [TensorSpec("wte.weight", (config.vocab_size, d), "table"),
               TensorSpec("wpe.weight", (config.n_positions, d), "table")]
    for i in range(config.n_layer):
        p = f"h.{i}."
        tensors += [
            TensorSpec(p + "ln_1.weight", (d,), "vector"), TensorSpec(p + "ln_1.bias", (d,), "vector"),
            TensorSpec(p + "attn.c_attn.weight", (d, 3 * d), "in_out"),
            TensorSpec(p + "attn.c_attn.bias", (3 * d,), "vector"),
            TensorSpec(p + "attn.c_proj.weight", (d, d), "in_out"),
            TensorSpec(p + "attn.c_proj.bias", (d,), "vector"),
            TensorSpec(p + "ln_2.weight", (d,), "vector"), TensorSpec(p + "ln_2.bias", (d,), "vector"),
            TensorSpec(p + "mlp.c_fc.weight", (d, m), "in_out"),
            TensorSpec(p + "mlp.c_fc.bias", (m,), "vector"),
            TensorSpec(p + "mlp.c_proj.weight", (m, d), "in_out"),
            TensorSpec(p + "mlp.c_proj.bias", (d,), "vector"),
        ]
    tensors += [TensorSpec("ln_f.weight", (d,), "vector"), TensorSpec("ln_f.bias", (d,), "vector")]
    return Contract(
        tensors=tensors,
        prefixes=("", "transformer."),           # backbone or language-model namespace
        anchor="wte.weight",
        # legacy causal-mask buffers of old checkpoints (src/models/gpt2/checkpoint.rs:169-174)
        ignored=(r"h\.\d+\.attn\.bias", r"h\.\d+\.attn\.masked_bias"),
        # a stored head must be the token table itself (checkpoint.rs:182-188)
        aliases={"lm_head.weight": "wte.weight"})


def init(config: GPT2Config, generator):
    s = config.initializer_range
    residual = s / math.sqrt(2.0 * config.n_layer)

    def normal(shape, std, mean=0.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32) * std + mean

    tensors = {}
    for spec in contract(config).tensors:
        name = spec.name
        if name.endswith("c_proj.weight"):
            tensors[name] = normal(spec.shape, residual)
        elif ".ln_" in name or name.startswith("ln_f."):
            tensors[name] = normal(spec.shape, s, 1.0 if name.endswith(".weight") else 0.0)
        else:
            tensors[name] = normal(spec.shape, s)
    return tensors


FAMILY = register_family(Family(
    name="gpt2", architectures=("GPT2LMHeadModel",), model_types=("gpt2",),
    config_class=GPT2Config, plan=plan, contract=contract, init=init))
