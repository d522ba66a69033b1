"""Normalisations over the channel axis, with 32-bit statistics in both precisions.

layer_norm: y = (x - mean) / sqrt(var + eps) * weight + bias, var the population variance
            (src/models/gpt2/model.rs:8, 143-148).
rms_norm:   y = x / sqrt(mean(x^2) + eps) * weight   (src/normalization.rs:158-171).

``apply`` first adds what is pending on the residual stream, in the same pass.
"""

from ..kernels import library as K
from .base import Norm
from .registry import register


class _KernelNorm(Norm):
    KIND = None
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.eps = params["width"], float(params["eps"])
        self.weight, self.bias = tensors["weight"], tensors.get("bias")
        if tuple(self.weight.shape) != (self.width,):
            raise ValueError(f"{self.KIND}: scale is {tuple(self.weight.shape)}, expected {(self.width,)}")

    def apply(self, stream, step, rows=None, chunked=False):
        count = rows.numel() if rows is not None else stream.x.shape[0]
        if chunked and K.Chunked.wanted(count) and self.width % 4 == 0:
            out = K.Chunked.take(step, "norm.out" if rows is None else "norm.selected", count, self.width, step.dtype)     # for a part that only hands it to `gemm`
        else:
            out = step.buffer("norm.out" if rows is None else "norm.selected", count, self.width, step.dtype)
        pending = stream.pending
        K.add_norm(stream.x, out, self.weight, self.bias, self.eps, self.KIND,
                   delta=pending.partials if pending else None, bias=pending.bias if pending else None,
                   rows=rows, write_back=rows is None)
        if rows is None:
            stream.pending = None
        return out

    def deferred_possible(self, step, rows):
        return step.dtype_is_bf16 and K.Normalized.worth_it(rows, self.width)

    def deferred(self, stream, step):
        if stream.pending is not None or not self.deferred_possible(step, stream.x.shape[0]):
            return None
        return K.Normalized(stream.x, self.weight, self.bias, self.eps, self.KIND)


@register("norm", "layer_norm")
class LayerNorm(_KernelNorm):
    KIND = "layer_norm"


@register("norm", "rms_norm")
class RMSNorm(_KernelNorm):
    KIND = "rms_norm"
