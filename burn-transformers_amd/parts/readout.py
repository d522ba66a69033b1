"""Readout: logits = h . table^T in float32, no bias; the table is [vocab, width] and may be
the token table itself (src/models/gpt2/model.rs:500-513, src/operations.rs:675-728)."""

from ..kernels import library as K
from .base import Readout
from .registry import register


@register("readout", "linear_readout")
class LinearReadout(Readout):
    only_launches_kernels = True
    takes_deferred_norm = True       # the rows are only handed to ``gemm``: the final norm may leave them chunk-major

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.weight = tensors["weight"]
        if tuple(self.weight.shape) != (self.vocab_size, self.width):
            raise ValueError(f"readout: table is {tuple(self.weight.shape)}, expected "
                             f"{(self.vocab_size, self.width)}")
        # a second copy for steps of few rows, which read the table and little else (the token
        # embedding looks rows up in the table as it is stored)
        self.packed = K.PackedWeight(self.weight) if self.weight.is_cuda else None

    def logits(self, h, step):
        out = step.buffer("readout.logits", h.shape[0], self.vocab_size, "float32")
        K.gemm(h, self.weight, K.epilogue_f32(out), packed=self.packed)
        return out
