"""Token embedding and position encodings that act at the embedding.

learned_positions: x0[t] = tokens[id[t]] + positions[pos[t]]  (src/models/gpt2/model.rs:447-448);
the table's length bounds a sequence's length.  token_only: x0[t] = tokens[id[t]] (for models
whose position encoding lives in the mixer).
"""

from ..kernels import library as K
from .base import Embedding, ResidualStream
from .registry import register


@register("embedding", "learned_positions")
class LearnedPositionEmbedding(Embedding):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.max_positions = params["max_positions"]
        self.token_table, self.position_table = tensors["tokens"], tensors["positions"]
        if tuple(self.token_table.shape) != (self.vocab_size, self.width) or \
                tuple(self.position_table.shape) != (self.max_positions, self.width):
            raise ValueError("embedding: tables do not have the configured sizes")

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        K.embed(step.tok_ids, step.tok_pos, self.token_table, self.position_table, x)
        return ResidualStream(x)


@register("embedding", "token_only")
class TokenEmbedding(Embedding):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.max_positions = params.get("max_positions", 2 ** 31 - 1)
        self.token_table = tensors["tokens"]

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        K.embed(step.tok_ids, None, self.token_table, None, x)
        return ResidualStream(x)
