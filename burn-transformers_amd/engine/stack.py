"""A model's whole schedule of layers as ONE kernel in small decode steps.

Where every layer of a model is the same arrangement (pre-norm block, causal attention over the
paged cache with a fused projection, dense feed-forward, the same kind of norm) and differs only
in its tensors and constants, a decode step of up to 16 sequences in bfloat16 does not have to be
five or six kernels a layer: ``csrc/decode_stack.hip`` keeps one work-group per compute unit
resident for all layers, with barriers across the grid between the phases of a layer and the
weights of a phase requested a phase or two ahead.  This file decides whether a model and a
step qualify, lays the layers' tensors out for the kernel, and launches it.  Everything else
(other parts, larger steps, float32, prompts) runs layer by layer through the parts themselves,
and so does a model whose sizes the kernel refuses.

It reads the parts' attributes; no part knows of it.
"""

import ctypes

import torch

from ..kernels import library as K
from ..parts.attention import CausalSelfAttention
from ..parts.base import compute_units
from ..parts.block import PreNormBlock
from ..parts.feed_forward import DenseFeedForward
from ..parts.norm import LayerNorm, RMSNorm


def columns_per_group(columns, groups, most):
    """Output columns a work-group owns of a product with ``columns`` of them: a multiple of four,
    at most ``most`` (one or two MFMA blocks of 16)."""
    return min(((columns + groups - 1) // groups + 3) // 4 * 4, most)


def pack_for_stack(weight, cols):
    """[N, K] -> [groups, chunks of 32 K values, cols, 32]: each group of ``cols`` output columns
    with its chunks of K one after the other, K and the last group padded with zeros.  A wave of
    the kernel then loads a chunk as one contiguous kilobyte, and a work-group reads its part of
    the matrix front to back."""
    n, k = weight.shape
    groups, chunks = (n + cols - 1) // cols, (k + 31) // 32
    padded = weight.new_zeros((groups * cols, chunks * 32))
    padded[:n, :k] = weight
    return padded.view(groups, cols, chunks, 32).permute(0, 2, 1, 3).contiguous()


def packed_layers(model, grid):
    """The four matrices of every layer in the kernel's layout, made once per model and grid size
    (a second copy of the layers' weights: the first stays as the other kernels read it)."""
    cache = model.__dict__.setdefault("_stack_packed", {})
    if grid not in cache:
        layers = []
        for entry in model.schedule:
            mixer, ff = model.blocks[entry.layer].parts["mixer"], model.blocks[entry.layer].parts["ff"]
            cols_qkv = columns_per_group(mixer.qkv_weight.shape[0], grid, 32)
            cols_up = columns_per_group(ff.up_weight.shape[0], grid, 32)
            cols_x = columns_per_group(mixer.out_weight.shape[0], grid, 16)
            layers.append(dict(cols=(cols_qkv, cols_up, cols_x),
                               qkv=pack_for_stack(mixer.qkv_weight, cols_qkv), out=pack_for_stack(mixer.out_weight, cols_x),
                               up=pack_for_stack(ff.up_weight, cols_up), down=pack_for_stack(ff.down_weight, cols_x)))
        cache[grid] = layers
    return cache[grid]


class DecodeStack:
    CHECK_EVERY = 256          # steps between two looks at the flag a barrier sets when its wait gave up

    def __init__(self, model, cache, shape, layers):
        self.model, self.cache, self.shape = model, cache, shape
        self.device = model.device
        self.grid = compute_units(self.device)
        self.packed = packed_layers(model, self.grid)
        self.cols = self.packed[0]["cols"]
        for layer, packed in zip(layers, self.packed):
            layer.qkv_weight, layer.out_weight = packed["qkv"].data_ptr(), packed["out"].data_ptr()
            layer.up_weight, layer.down_weight = packed["up"].data_ptr(), packed["down"].data_ptr()
        table = (K.StackLayer * len(layers))(*layers)
        self.layers = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8).to(self.device)
        self.sync, self.failed_word = K.decode_stack_sync(shape["head_dim"], self.device)
        self.clocks = None             # see ``record_clocks``
        self.refused = None            # the kernel's message once it has refused this model's sizes
        self.launches = 0
        self._unchecked = 0

    # --- does the model qualify? ---------------------------------------------------------------
    @classmethod
    def build(cls, model, cache):
        """The stack of a model and its cache, or None where the layers are not all of the one
        arrangement the kernel implements."""
        if model.dtype != torch.bfloat16 or not model.schedule:
            return None
        shape, layers, seen = None, [], set()
        for entry in model.schedule:
            block = model.blocks[entry.layer]
            if type(block) is not PreNormBlock or entry.cache is None or not entry.writes or entry.cache in seen:
                return None
            seen.add(entry.cache)
            mixer, ff = block.parts["mixer"], block.parts["ff"]
            norm1, norm2 = block.parts["mixer_norm"], block.parts["ff_norm"]
            if type(mixer) is not CausalSelfAttention or type(ff) is not DenseFeedForward:
                return None
            if type(norm1) not in (LayerNorm, RMSNorm) or type(norm2) is not type(norm1):
                return None
            this = dict(width=mixer.width, heads=mixer.heads, kv_heads=mixer.kv_heads, head_dim=mixer.head_dim,
                        window=mixer.window, inner=ff.padded, activation=ff.activation, norm=norm1.KIND)
            if ff.width != mixer.width or norm1.width != mixer.width or norm2.width != mixer.width:
                return None
            if shape is None:
                shape = this
            elif this != shape:
                return None
            if entry.cache not in cache.kv_entry:
                return None
            group, index = cache.kv_entry[entry.cache]
            if group != cache.kv_entry[model.schedule[0].cache][0]:
                return None
            store = cache.kv_groups[group]
            layers.append(K.StackLayer(
                norm1_scale=K._ptr(norm1.weight), norm1_shift=K._ptr(norm1.bias),
                norm2_scale=K._ptr(norm2.weight), norm2_shift=K._ptr(norm2.bias),
                qkv_weight=K._ptr(mixer.qkv_weight), qkv_bias=K._ptr(mixer.qkv_bias),
                out_weight=K._ptr(mixer.out_weight), out_bias=K._ptr(mixer.out_bias),
                up_weight=K._ptr(ff.up_weight), up_bias=K._ptr(ff.up_bias),
                down_weight=K._ptr(ff.down_weight), down_bias=K._ptr(ff.down_bias),
                keys=store.keys[index].data_ptr(), values=store.values[index].data_ptr(),
                eps1=norm1.eps, eps2=norm2.eps, scale=mixer.scale, reserved=0))
        if shape["head_dim"] > 128:
            return None
        return cls(model, cache, shape, layers)

    def takes(self, step):
        return (self.refused is None and step.decode and step.dtype_is_bf16
                and 0 < step.n_seqs <= K.STACK_MAX_ROWS and step.n_tokens == step.n_seqs)

    # --- one step ------------------------------------------------------------------------------
    def run(self, stream, step):
        """Runs every layer on the residual stream in place.  False if the kernel refuses the
        model's sizes (nothing has run then, and it is not asked again)."""
        s = self.shape
        rows, n_q, layers = step.n_seqs, s["heads"] * s["head_dim"], len(self.model.schedule)
        stream.flush()
        # every layer has a place of its own in the exchange buffers, a whole number of 256-byte units
        place = lambda elements, size: (elements * size + 255) // 256 * 256 // size
        args = K.StackArgs(
            layers=self.layers.data_ptr(), n_layers=layers, rows=rows,
            x=stream.x.data_ptr(), ldx=stream.x.stride(0), width=s["width"], inner=s["inner"],
            heads=s["heads"], kv_heads=s["kv_heads"], norm_kind=K.NORM_KINDS[s["norm"]],
            act=K.ACTIVATIONS[s["activation"]], window=s["window"], max_blocks=step.max_blocks,
            cols_qkv=self.cols[0], cols_up=self.cols[1], cols_x=self.cols[2],
            blocks=step.block_table.data_ptr(), positions=step.seq_start.data_ptr(),
            q=step.buffer("stack.q", layers, place(rows * n_q, 2), step.dtype).data_ptr(),
            mixed=step.buffer("stack.mixed", layers, place(rows * n_q, 2), step.dtype).data_ptr(),
            hidden=step.buffer("stack.hidden", layers, place(rows * s["inner"], 2), step.dtype).data_ptr(),
            between=step.buffer("stack.between", 2 * layers, place(rows * s["width"], 4), "float32").data_ptr(),
            sync=self.sync.data_ptr(), clocks=K._ptr(self.clocks))
        self.sync[:self.failed_word].zero_()          # a fill kernel (also under graph capture); the flag stays
        try:
            K.decode_stack(s["head_dim"], args, self.grid)
        except K.KernelError as error:
            self.refused = str(error)
            return False
        self.launches += 1
        self._unchecked += 1
        return True

    def record_clocks(self):
        """From now on every launch leaves when the phases of its first layers began and ended:
        int64 [work-groups, layers, 10] ticks of the 100 MHz wall clock, (begin, end) of the fused
        projection, attention, output projection, feed-forward in, feed-forward out."""
        layers = K.decode_stack_module(self.shape["head_dim"]).bt_decode_stack_clock_layers()
        self.clocks = torch.zeros((self.grid, layers, 10), dtype=torch.int64, device=self.device)
        return self.clocks

    def check(self, force=False):
        """Raises if a barrier of an earlier launch gave up waiting (its work-groups were not all
        resident at once); looked at every CHECK_EVERY steps and when asked."""
        if self._unchecked == 0 or (not force and self._unchecked < self.CHECK_EVERY):
            return
        self._unchecked = 0
        if int(self.sync[self.failed_word]) != 0:
            raise RuntimeError("decode_stack: a barrier across the grid gave up waiting; the results of "
                               "decode steps since the last check are invalid")
