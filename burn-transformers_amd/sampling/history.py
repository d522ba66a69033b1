"""What history-dependent processing of the logits needs of each row (TokenHistory,
src/generation/history.rs:1-60, 446-530): how often every token has occurred, on the GPU and
updated with each step's new tokens; the n-grams of prompt and output and the generated length,
on the host.

  counts_all[row][token]        occurrences in prompt and output  (repetition penalty; additive
                                penalties with scope "prompt_and_generated")
  counts_generated[row][token]  occurrences in the output         (additive penalties, default scope)
  banned(row)                   tokens that would complete an n-gram of size no_repeat_ngram_size
                                that the row already holds (src/generation/ngram.rs:1-12), plus the
                                end-of-sequence ids while the row is below min_new_tokens
                                (src/generation.rs:757-761)
"""

import torch

from ..kernels import library as K


class NgramIndex:
    """Followers of every (n - 1)-token prefix of one row; pure Python."""

    def __init__(self, size):
        self.size, self.tokens, self.followers = size, [], {}

    def push(self, token):
        self.tokens.append(token)
        n = self.size
        if len(self.tokens) >= n:                      # the newest token completes an n-gram
            prefix = tuple(self.tokens[len(self.tokens) - n:len(self.tokens) - 1])
            self.followers.setdefault(prefix, set()).add(token)

    def banned(self):
        """Tokens that may not come next: they followed the last n - 1 tokens before."""
        n = self.size
        if len(self.tokens) < n - 1:
            return []
        prefix = tuple(self.tokens[len(self.tokens) - (n - 1):]) if n > 1 else ()
        return sorted(self.followers.get(prefix, ()))


class TokenHistory:
    def __init__(self, config, vocabulary_size, prompts, device):
        self.config, self.vocabulary_size, self.device = config, vocabulary_size, device
        rows = len(prompts)
        self.generated_lengths = [0] * rows
        self.ngrams = None
        if config.no_repeat_ngram_size > 0:
            self.ngrams = [NgramIndex(config.no_repeat_ngram_size) for _ in prompts]
            for index, prompt in zip(self.ngrams, prompts):
                for token in prompt:
                    index.push(token)
        self.counts_all = self.counts_generated = None
        if config.counts_all:
            self.counts_all = torch.zeros((rows, vocabulary_size), dtype=torch.int32, device=device)
            pairs = [(row, token) for row, prompt in enumerate(prompts) for token in prompt]
            if pairs:
                K.count_tokens(self.counts_all, [r for r, _ in pairs], [t for _, t in pairs])
        if config.counts_generated:
            self.counts_generated = torch.zeros((rows, vocabulary_size), dtype=torch.int32, device=device)

    @property
    def additive_counts(self):
        return self.counts_generated if self.config.counts_generated else \
            (self.counts_all if (self.config.presence_penalty != 0.0 or self.config.frequency_penalty != 0.0) else None)

    def banned(self, row):
        tokens = self.ngrams[row].banned() if self.ngrams is not None else []
        if self.config.eos_token_ids and self.generated_lengths[row] < self.config.min_new_tokens:
            tokens = sorted(set(tokens) | set(self.config.eos_token_ids))
        return tokens

    def record(self, rows, tokens):
        """The rows' newly generated tokens (one each)."""
        for row, token in zip(rows, tokens):
            self.generated_lengths[row] += 1
            if self.ngrams is not None:
                self.ngrams[row].push(token)
        if rows and self.counts_all is not None:
            K.count_tokens(self.counts_all, rows, tokens)
        if rows and self.counts_generated is not None:
            K.count_tokens(self.counts_generated, rows, tokens)
