"""Controls of generation, with the reference's names, defaults and meanings
(GenerationConfig, src/generation.rs:191-276)."""

import math
import struct
from dataclasses import dataclass, field
from typing import Dict, List, Optional

F32_MIN_NORMAL, F32_MAX = 1.1754943508222875e-38, 3.4028234663852886e38


class GenerationError(ValueError):
    """A generation request is invalid or a step produced a non-finite log-probability."""


def _as_f32(value):
    """``value`` rounded to float32 the way a kernel argument is (inf when it overflows)."""
    try:
        return struct.unpack("f", struct.pack("f", float(value)))[0]
    except OverflowError:
        return math.copysign(math.inf, value)


def _check_divisor(name, value):
    """A divisor must round to a normal positive float32 (src/generation.rs:1033-1056)."""
    rounded = _as_f32(value) if isinstance(value, (int, float)) and not isinstance(value, bool) else math.nan
    if not (math.isfinite(rounded) and F32_MIN_NORMAL <= rounded <= F32_MAX):
        raise GenerationError(f"{name} must round to a normal positive F32 value in "
                              f"{F32_MIN_NORMAL:.8e}..={F32_MAX:.8e}, found {value}")


def _check_finite(name, value):
    """An additive control must round to a finite float32 (src/generation.rs:1058-1075)."""
    rounded = _as_f32(value) if isinstance(value, (int, float)) and not isinstance(value, bool) else math.nan
    if not math.isfinite(rounded):
        raise GenerationError(f"{name} must round to a finite F32 value (at most {F32_MAX:.8e} in magnitude), "
                              f"found {value}")


@dataclass
class GenerationConfig:
    max_new_tokens: int = 256
    min_new_tokens: int = 0            # end-of-sequence is banned and stop sequences are ignored until reached
    strategy: str = "greedy"           # "greedy" or "sample"
    temperature: float = 1.0           # divides the logits only when sampling
    top_k: Optional[int] = None        # sampling: keep scores >= the k-th greatest (ties survive)
    top_p: Optional[float] = None      # sampling: keep the shortest prefix of the ranking whose mass reaches p
    min_p: Optional[float] = None      # sampling: keep p_i >= min_p * max p
    repetition_penalty: float = 1.0    # z / r (z * r below zero) for every token of prompt or output
    presence_penalty: float = 0.0      # subtracted once from every token the scope has counted
    frequency_penalty: float = 0.0     # subtracted per occurrence the scope has counted
    additive_penalty_scope: str = "generated"   # or "prompt_and_generated"
    no_repeat_ngram_size: int = 0      # no n-gram of prompt + output may occur twice; 0 disables
    logit_bias: Dict[int, float] = field(default_factory=dict)   # added before the penalties
    seed: int = 0                      # SplitMix64 stream of the uniform draws
    eos_token_ids: List[int] = field(default_factory=list)   # emitted, then the sequence ends
    pad_token_id: Optional[int] = None
    stop_sequences: List[List[int]] = field(default_factory=list)

    def validate(self, vocabulary_size):
        """Names the first invalid field, in the reference's order (src/generation.rs:278-405)."""
        if vocabulary_size <= 0:
            raise GenerationError("vocabulary_size must be greater than zero")
        if self.max_new_tokens <= 0:
            raise GenerationError("max_new_tokens must be greater than zero")
        if self.min_new_tokens < 0 or self.min_new_tokens > self.max_new_tokens:
            raise GenerationError(f"min_new_tokens {self.min_new_tokens} exceeds max_new_tokens {self.max_new_tokens}"
                                  if self.min_new_tokens >= 0 else "min_new_tokens must not be negative")
        if self.strategy not in ("greedy", "sample"):
            raise GenerationError(f"strategy must be `greedy` or `sample`, got `{self.strategy}`")
        # sampling controls
        _check_divisor("temperature", self.temperature)
        if self.top_k is not None and not (isinstance(self.top_k, int) and 1 <= self.top_k <= vocabulary_size):
            raise GenerationError(f"top_k must be in 1..={vocabulary_size}, found {self.top_k}")
        if self.top_p is not None and not (math.isfinite(self.top_p) and 0.0 < self.top_p <= 1.0):
            raise GenerationError(f"top_p must be finite and in (0, 1], found {self.top_p}")
        if self.min_p is not None and not (0.0 <= self.min_p <= 1.0):
            raise GenerationError(f"min_p must be in [0, 1], found {self.min_p}")
        # penalties
        _check_divisor("repetition_penalty", self.repetition_penalty)
        _check_finite("presence_penalty", self.presence_penalty)
        _check_finite("frequency_penalty", self.frequency_penalty)
        if self.additive_penalty_scope not in ("generated", "prompt_and_generated"):
            raise GenerationError("additive_penalty_scope must be `generated` or `prompt_and_generated`, "
                                  f"got `{self.additive_penalty_scope}`")
        if not (isinstance(self.no_repeat_ngram_size, int) and self.no_repeat_ngram_size >= 0):
            raise GenerationError("no_repeat_ngram_size must not be negative")
        if not (0 <= self.seed < 2 ** 64):
            raise GenerationError("seed must fit 64 bits")
        # token ids: end-of-sequence, padding, stop sequences, then the biased tokens
        special = list(self.eos_token_ids) + ([self.pad_token_id] if self.pad_token_id is not None else [])
        for sequence in self.stop_sequences:
            special += list(sequence)
        for token in special:
            if not (0 <= token < vocabulary_size):
                raise GenerationError(f"special token {token} is outside vocabulary size {vocabulary_size}")
        if any(len(sequence) == 0 for sequence in self.stop_sequences):
            raise GenerationError("stop sequences must not be empty")
        for token in sorted(self.logit_bias):
            if not (isinstance(token, int) and 0 <= token < vocabulary_size):
                raise GenerationError(f"logit_bias token {token} is outside vocabulary size {vocabulary_size}")
            _check_finite(f"logit_bias for token {token}", self.logit_bias[token])

    @property
    def sampling(self):
        return self.strategy == "sample"

    @property
    def adjusts_logits(self):
        """Bias or a penalty changes logits arithmetically, and so can overflow (generation.rs:362-368)."""
        return bool(self.logit_bias) or self.repetition_penalty != 1.0 or self.presence_penalty != 0.0 or \
            self.frequency_penalty != 0.0

    @property
    def counts_all(self):
        """Some penalty reads the counts of prompt and output together (generation.rs:418-425)."""
        additive = self.presence_penalty != 0.0 or self.frequency_penalty != 0.0
        return self.repetition_penalty != 1.0 or (additive and self.additive_penalty_scope == "prompt_and_generated")

    @property
    def counts_generated(self):
        additive = self.presence_penalty != 0.0 or self.frequency_penalty != 0.0
        return additive and self.additive_penalty_scope == "generated"

    def truncates(self, vocabulary_size):
        """A warper that is switched on and not a no-op (generation.rs:926-948)."""
        return self.sampling and ((self.top_k is not None and self.top_k < vocabulary_size) or
                                  (self.top_p is not None and self.top_p < 1.0) or
                                  (self.min_p is not None and self.min_p > 0.0))

    def processes_logits(self, vocabulary_size):
        """Anything beyond plain greedy selection or plain temperature sampling is asked for."""
        return self.adjusts_logits or self.no_repeat_ngram_size > 0 or \
            (self.min_new_tokens > 0 and bool(self.eos_token_ids)) or self.truncates(vocabulary_size)
