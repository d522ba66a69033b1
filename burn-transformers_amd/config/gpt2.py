"""GPT-2's typed configuration, read from the keys of its own config.json.

Field names, aliases, defaults and the order of validation follow the reference
(src/models/gpt2.rs:105-171 and 258-318).  Unknown keys are ignored; every key is optional.
"""

from dataclasses import dataclass
from typing import Optional

from .base import (ConfigError, MAX_LAYERS, positive_extent, positive_finite, take,
                   unwrap_text_config)

FAMILY = "gpt2"
ACTIVATIONS = ("gelu_new", "gelu")


@dataclass(frozen=True)
class GPT2Config:
    model_type: str = "gpt2"
    vocab_size: int = 50257
    n_embd: int = 768
    n_layer: int = 12
    n_head: int = 12
    n_positions: int = 1024
    n_inner: Optional[int] = None
    activation_function: str = "gelu_new"
    layer_norm_epsilon: float = 1e-5
    scale_attn_weights: bool = True
    scale_attn_by_inverse_layer_idx: bool = False
    reorder_and_upcast_attn: bool = False
    add_cross_attention: bool = False
    tie_word_embeddings: bool = True
    causal: bool = True
    initializer_range: float = 0.02

    @property
    def intermediate_size(self):
        """n_inner, or four times the width when it is absent (src/models/gpt2/extents.rs:86-105)."""
        return self.n_inner if self.n_inner is not None else 4 * self.n_embd

    @property
    def head_size(self):
        return self.n_embd // self.n_head

    @classmethod
    def from_dict(cls, data):
        data = unwrap_text_config(data)
        config = cls(
            model_type=take(data, FAMILY, "model_type", str, "gpt2"),
            vocab_size=take(data, FAMILY, "vocab_size", int, 50257),
            n_embd=take(data, FAMILY, "n_embd", int, 768, ("hidden_size",)),
            n_layer=take(data, FAMILY, "n_layer", int, 12, ("num_hidden_layers",)),
            n_head=take(data, FAMILY, "n_head", int, 12, ("num_attention_heads",)),
            n_positions=take(data, FAMILY, "n_positions", int, 1024, ("max_position_embeddings",)),
            n_inner=take(data, FAMILY, "n_inner", int, None),
            activation_function=take(data, FAMILY, "activation_function", str, "gelu_new"),
            layer_norm_epsilon=take(data, FAMILY, "layer_norm_epsilon", float, 1e-5),
            scale_attn_weights=take(data, FAMILY, "scale_attn_weights", bool, True),
            scale_attn_by_inverse_layer_idx=take(data, FAMILY, "scale_attn_by_inverse_layer_idx", bool, False),
            reorder_and_upcast_attn=take(data, FAMILY, "reorder_and_upcast_attn", bool, False),
            add_cross_attention=take(data, FAMILY, "add_cross_attention", bool, False),
            tie_word_embeddings=take(data, FAMILY, "tie_word_embeddings", bool, True),
            causal=take(data, FAMILY, "causal", bool, True),
            initializer_range=take(data, FAMILY, "initializer_range", float, 0.02),
        )
        config.validate()
        return config

    def validate(self):
        """Same checks in the same order as the reference, so the first bad field is the one named
        (src/models/gpt2.rs:258-318)."""
        if self.activation_function not in ACTIVATIONS:   # a closed enum: fails while parsing
            raise ConfigError(FAMILY, "activation_function",
                              f"unknown variant `{self.activation_function}`, expected one of `gelu`, `gelu_new`")
        if self.model_type != "gpt2":
            raise ConfigError(FAMILY, "model_type", f"expected `gpt2`, got `{self.model_type}`")
        for field in ("vocab_size", "n_embd", "n_layer", "n_head", "n_positions"):
            positive_extent(FAMILY, field, getattr(self, field))
        if self.n_layer > MAX_LAYERS:
            raise ConfigError(FAMILY, "n_layer", f"must not exceed {MAX_LAYERS}")
        if self.n_embd % self.n_head != 0:
            raise ConfigError(FAMILY, "n_head", "must divide n_embd")
        positive_finite(FAMILY, "layer_norm_epsilon", self.layer_norm_epsilon)
        positive_finite(FAMILY, "initializer_range", self.initializer_range)
        if self.reorder_and_upcast_attn:
            raise ConfigError(FAMILY, "reorder_and_upcast_attn",
                              "the reordered, upcast attention graph is not implemented")
        if self.add_cross_attention:
            raise ConfigError(FAMILY, "add_cross_attention", "cross-attention blocks are not implemented")
        if not self.tie_word_embeddings:
            raise ConfigError(FAMILY, "tie_word_embeddings", "the readout must be tied to the token embedding")
        if not self.causal:
            # the reference's stateless module can run unmasked (src/models/gpt2.rs:141); a cached
            # step cannot: a token's keys would have to include tokens that are not there yet
            raise ConfigError(FAMILY, "causal", "only causal attention can run from a cache")
        if self.n_inner is not None and not (0 < self.n_inner <= 2 ** 62):
            raise ConfigError(FAMILY, "n_inner", "must be positive and fit usize")
        for width in (self.vocab_size, self.n_positions, self.intermediate_size, 3):
            if self.n_embd * width >= 2 ** 63:
                raise ConfigError(FAMILY, "n_embd", "parameter dimensions overflow usize")

    def to_dict(self):
        data = {field: getattr(self, field) for field in self.__dataclass_fields__}
        data["architectures"] = ["GPT2LMHeadModel"]
        return data
