"""Per-sequence bookkeeping of a generation: emitted tokens, log-probabilities and why a
sequence ended.  Pure Python; the generation loop asks it after every token.

Rules (src/generation.rs:1277-1422, src/generation/bookkeeping.rs:177-296):
  * an end-of-sequence token is emitted, then the sequence ends (EndOfSequence);
  * otherwise the longest stop sequence that is a suffix of the emitted tokens ends it
    (StopSequence; ties go to the first configured); the matched tokens stay emitted;
  * otherwise reaching max_new_tokens ends it (Length);
  * before min_new_tokens neither end-of-sequence nor stop sequences are looked at.
A sequence may have a limit of its own below max_new_tokens (a batch of unequal prompts that
all grow to one total length); the reference has one limit for the whole batch.
"""

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class FinishReason:
    kind: str                          # "eos", "stop" or "length"
    token_id: Optional[int] = None     # eos
    index: Optional[int] = None        # stop: which configured sequence
    length: Optional[int] = None       # stop: its length

    def __str__(self):
        if self.kind == "eos":
            return f"EndOfSequence(token_id={self.token_id})"
        if self.kind == "stop":
            return f"StopSequence(index={self.index}, length={self.length})"
        return "Length"


@dataclass
class GeneratedSequence:
    prompt_length: int
    token_ids: List[int] = field(default_factory=list)
    log_probabilities: List[float] = field(default_factory=list)
    finish_reason: Optional[FinishReason] = None


def stop_decision(config, emitted, limit=None):
    """Why a sequence whose emitted tokens are ``emitted`` ends now, or None.  ``limit`` is the
    sequence's own bound on new tokens where it has one (never above max_new_tokens)."""
    count = len(emitted)
    if count >= config.min_new_tokens:
        if emitted and emitted[-1] in config.eos_token_ids:
            return FinishReason("eos", token_id=emitted[-1])
        best = None
        for index, sequence in enumerate(config.stop_sequences):
            n = len(sequence)
            if n <= count and emitted[count - n:] == list(sequence) and (best is None or n > best[1]):
                best = (index, n)
        if best is not None:
            return FinishReason("stop", index=best[0], length=best[1])
    if count >= (config.max_new_tokens if limit is None else min(limit, config.max_new_tokens)):
        return FinishReason("length")
    return None


class GenerationTracker:
    def __init__(self, config, prompt_lengths, limits=None):
        self.config = config
        self.sequences = [GeneratedSequence(n) for n in prompt_lengths]
        self.limits = list(limits) if limits is not None else [None] * len(self.sequences)

    def push(self, row, token, log_probability):
        """Records a token of a live row; returns its finish reason if it ends now."""
        sequence = self.sequences[row]
        if sequence.finish_reason is not None:
            raise RuntimeError(f"row {row} has already finished")
        sequence.token_ids.append(int(token))
        sequence.log_probabilities.append(float(log_probability))
        sequence.finish_reason = stop_decision(self.config, sequence.token_ids, self.limits[row])
        return sequence.finish_reason

    def limit(self, row):
        """The most new tokens the row may get."""
        own = self.limits[row]
        return self.config.max_new_tokens if own is None else min(own, self.config.max_new_tokens)

    def finished(self, row):
        return self.sequences[row].finish_reason is not None

    def live_rows(self):
        return [i for i, s in enumerate(self.sequences) if s.finish_reason is None]

    def all_finished(self):
        return all(s.finish_reason is not None for s in self.sequences)


def required_capacity(prompt_length, max_new_tokens):
    """Positions a sequence occupies: the last generated token is returned but never fed back
    (src/generation/bookkeeping.rs:736-747)."""
    return prompt_length + max_new_tokens - 1
