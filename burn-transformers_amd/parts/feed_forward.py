"""Dense feed-forward: down(act(up(x)))  (src/feed_forward.rs:111-114).

Parameters: width, inner, activation ("gelu_tanh": 0.5x(1+tanh(sqrt(2/pi)(x+0.044715x^3))),
"gelu_erf": x(1+erf(x/sqrt 2))/2; src/feed_forward.rs:351-387).  The activation runs in 32-bit
inside the up projection's epilogue (src/feed_forward.rs:397-406 widens half inputs too); the
down projection adds into the residual stream.

The MFMA kernels read operands 16 bytes at a time, so an inner width that is no multiple of 8 is
padded once, when the part is built: zero rows (and zero bias) in the up projection give
act(0) = 0 in the padded columns, which meet zero columns of the down projection.
"""

import torch

from ..kernels import library as K
from .base import FeedForward, packed_for_stream
from .registry import register


@register("feed_forward", "dense")
class DenseFeedForward(FeedForward):
    takes_deferred_norm = True
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.inner, self.activation = params["width"], params["inner"], params["activation"]
        if self.activation not in K.ACTIVATIONS:
            raise ValueError(f"feed-forward: unknown activation {self.activation!r}")
        self.up_weight, self.up_bias = tensors["up_weight"], tensors.get("up_bias")
        self.down_weight, self.down_bias = tensors["down_weight"], tensors.get("down_bias")
        if tuple(self.up_weight.shape) != (self.inner, self.width) or \
                tuple(self.down_weight.shape) != (self.width, self.inner):
            raise ValueError(f"feed-forward: projections are {tuple(self.up_weight.shape)} and "
                             f"{tuple(self.down_weight.shape)}, expected {(self.inner, self.width)} and "
                             f"{(self.width, self.inner)}")
        self.padded = (self.inner + 7) // 8 * 8
        extra = self.padded - self.inner
        if extra:
            up, down = self.up_weight, self.down_weight
            self.up_weight = torch.cat([up, up.new_zeros(extra, self.width)]).contiguous()
            self.down_weight = torch.cat([down, down.new_zeros(self.width, extra)], dim=1).contiguous()
            if self.up_bias is not None:
                self.up_bias = torch.cat([self.up_bias, self.up_bias.new_zeros(extra)]).contiguous()

        # second copies for decode steps, which read the weights and little else
        self.up_packed = K.PackedWeight(self.up_weight) if self.up_weight.is_cuda else None
        self.down_packed = packed_for_stream(self.down_weight) if self.down_weight.is_cuda else None

    def forward(self, h, step, stream):
        tokens = h.shape[0]
        if K.Chunked.wanted(tokens) and (step.dtype_is_bf16 or self.padded % 4 == 0):
            hidden = K.Chunked.take(step, "feed_forward.hidden", tokens, self.padded, step.dtype)   # read by the next product only
        else:
            hidden = step.buffer("feed_forward.hidden", tokens, self.padded, step.dtype)
        K.gemm(h, self.up_weight, K.epilogue_act(hidden, self.activation, self.up_bias), packed=self.up_packed)
        stream.add_product(step, hidden, self.down_weight, self.down_bias, packed=self.down_packed)
