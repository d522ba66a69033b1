"""Controls of generation, with the reference's names, defaults and meanings
(GenerationConfig, src/generation.rs:191-276)."""

import math
from dataclasses import dataclass, field
from typing import List, Optional

# options of the reference that this library does not build; setting one is an error, not a no-op
NOT_BUILT = ("top_k", "top_p", "min_p", "repetition_penalty", "presence_penalty", "frequency_penalty",
             "no_repeat_ngram_size", "logit_bias")


class GenerationError(ValueError):
    """A generation request is invalid or a step produced a non-finite log-probability."""


@dataclass
class GenerationConfig:
    max_new_tokens: int = 256
    min_new_tokens: int = 0            # end-of-sequence and stop sequences are ignored until reached
    strategy: str = "greedy"           # "greedy" or "sample"
    temperature: float = 1.0           # divides the logits only when sampling
    seed: int = 0                      # SplitMix64 stream of the uniform draws
    eos_token_ids: List[int] = field(default_factory=list)   # emitted, then the sequence ends
    pad_token_id: Optional[int] = None
    stop_sequences: List[List[int]] = field(default_factory=list)
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    min_p: Optional[float] = None
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    no_repeat_ngram_size: int = 0
    logit_bias: dict = field(default_factory=dict)

    def validate(self, vocabulary_size):
        """Names the first invalid field (src/generation.rs:288 ff.)."""
        if vocabulary_size <= 0:
            raise GenerationError("vocabulary_size must be greater than zero")
        if self.max_new_tokens <= 0:
            raise GenerationError("max_new_tokens must be greater than zero")
        if self.min_new_tokens > self.max_new_tokens:
            raise GenerationError("min_new_tokens must not exceed max_new_tokens")
        if self.strategy not in ("greedy", "sample"):
            raise GenerationError(f"strategy must be `greedy` or `sample`, got `{self.strategy}`")
        t = float(self.temperature)
        if not (math.isfinite(t) and 1.1754944e-38 <= t <= 3.4028235e38):
            raise GenerationError("temperature must round to a normal positive F32 value")
        if not (0 <= self.seed < 2 ** 64):
            raise GenerationError("seed must fit 64 bits")
        for token in self.eos_token_ids:
            if not (0 <= token < vocabulary_size):
                raise GenerationError(f"eos_token_ids entry {token} is outside the vocabulary")
        if self.pad_token_id is not None and not (0 <= self.pad_token_id < vocabulary_size):
            raise GenerationError(f"pad_token_id {self.pad_token_id} is outside the vocabulary")
        for sequence in self.stop_sequences:
            if not sequence:
                raise GenerationError("stop_sequences must not contain an empty sequence")
            for token in sequence:
                if not (0 <= token < vocabulary_size):
                    raise GenerationError(f"stop_sequences token {token} is outside the vocabulary")
        defaults = GenerationConfig()
        for name in NOT_BUILT:
            if getattr(self, name) != getattr(defaults, name):
                raise GenerationError(f"{name} is not built in this library (greedy and temperature sampling are)")

    @property
    def sampling(self):
        return self.strategy == "sample"
