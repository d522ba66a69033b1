"""Tiny configurations and helpers shared by the engine tests."""

import json
import os
import tempfile

import torch

import burn_transformers_amd as bt
import plain_gpt2 as plain

# Two tiny GPT-2 configurations that differ in every size and option.
TINY_A = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 64, "n_head": 4,
          "n_inner": 256, "vocab_size": 1000, "n_positions": 128, "activation_function": "gelu_new",
          "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
TINY_B = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 3, "n_embd": 96, "n_head": 2,
          "n_inner": 320, "vocab_size": 517, "n_positions": 64, "activation_function": "gelu",
          "layer_norm_epsilon": 1e-6, "scale_attn_by_inverse_layer_idx": True}
# the same with room for sequences that cross several blocks of the cache
TINY_BW = dict(TINY_B, n_positions=192)
# an inner width that is odd, one head size, one layer: sizes the 16-byte loads of the kernels do not divide
TINY_C = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 1, "n_embd": 32, "n_head": 2,
          "n_inner": 37, "vocab_size": 131, "n_positions": 80, "activation_function": "gelu_new",
          "layer_norm_epsilon": 1e-3, "scale_attn_by_inverse_layer_idx": False}
# room for contexts of several thousand tokens: decode steps there cut the keys into runs
TINY_L = {"architectures": ["GPT2LMHeadModel"], "model_type": "gpt2", "n_layer": 2, "n_embd": 96, "n_head": 3,
          "n_inner": 128, "vocab_size": 211, "n_positions": 4300, "activation_function": "gelu_new",
          "layer_norm_epsilon": 1e-5, "scale_attn_by_inverse_layer_idx": False}
CONFIGS = {"A": (TINY_A, 0), "B": (TINY_B, 1), "BW": (TINY_BW, 1), "C": (TINY_C, 2), "L": (TINY_L, 3)}

_folders = {}


def model_folder(name, gain=1.0):
    """(folder, config, float32 weights as stored) of a tiny random model; made once per process in
    a temporary folder.  ``gain`` scales every matrix, which makes logits less uniform."""
    key = (name, gain)
    if key not in _folders:
        config, seed = CONFIGS[name]
        holder = tempfile.TemporaryDirectory(prefix=f"bt_tiny_{name}_")
        weights = bt.write_random_model(holder.name, config, seed)
        if gain != 1.0:
            weights = {k: (v * gain if v.dim() == 2 else v) for k, v in weights.items()}
            bt.write_safetensors(os.path.join(holder.name, "model.safetensors"),
                                 {k: v.to(torch.bfloat16) for k, v in weights.items()})
            weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
        _folders[key] = (holder, config, weights)
    holder, config, weights = _folders[key]
    return holder.name, config, weights


def plain_logits(name, ids, gain=1.0):
    """float64 logits [len(ids), vocab] of the plain implementation."""
    _, config, weights = model_folder(name, gain)
    return plain.forward(ids, weights, config)


def prompts_for(name, lengths, seed=0):
    config, _ = CONFIGS[name]
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, config["vocab_size"], (n,), generator=gen).tolist() for n in lengths]


def tolerance(dtype, reference):
    """Largest allowed absolute error of logits: float32 differs from float64 by summation order
    only; bfloat16 rounds every activation between two kernels to 8 bits of mantissa (relative
    2^-9 = 2e-3 each), which through the few layers of these models measures 2e-3 to 4e-3 of the
    largest logit; the bound is twice that."""
    scale = float(reference.abs().max())
    return 2e-5 + 1e-5 * scale if dtype == "float32" else 8e-3 * scale
