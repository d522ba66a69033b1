"""Causal self-attention with grouped heads over the paged cache.

Parameters (all from the plan): width, heads, kv_heads, head_dim, scale (multiplies q.k),
window (0 = every earlier key), causal.  Tensors: a fused projection ``qkv_weight`` held
[heads*head_dim + 2*kv_heads*head_dim, width] with its bias, and ``out_weight`` [width,
heads*head_dim] with its bias.

One step: the fused projection's epilogue writes the queries to a buffer and scatters the new
keys and values straight into the cache at each token's position; the attention kernel then
reads the cache (prefill: tiled, online softmax; decode: one query per head, keys split over
the waves, and long contexts of a small batch over several work-groups); the output projection
adds into the residual stream.
Formulas: src/attention.rs:481-513 (projections), src/attention/dispatch.rs:314-328, 365-367,
390-406 (scaled scores, exclusion by -inf, 32-bit softmax), src/attention.rs:882-897 (merge and
output projection).
"""

import torch

from ..cache.storage import KVSpec
from ..kernels import library as K
from .base import Mixer, compute_units, packed_for_stream
from .registry import register

# A decode step cuts long contexts into runs that separate work-groups take and a second kernel
# joins.  Measured at 25 heads of 64 (us per call, runs 1 / 2 / 4 / 8 / 16): bfloat16, one
# sequence, 1,024 keys 9.1 / 9.4 / 9.6 / 11.5 / 15.2, 2,048 keys 14.5 / 12.2 / 10.9 / 12.4 / 16.8,
# 8,192 keys 47.7 / 29.6 / 23.0 / 19.3 / 23.6; eight sequences (200 pairs of sequence and head
# already) lose with any cut, 73 / 80 / 85 us at 8,192 keys.  So: no more work-groups than
# compute units, at least RUN_BYTES of keys and values per run, and no cut below SPLIT_BYTES.
# (With the joining kernel that asks for eight runs' records at once, one sequence measures 7.1 us
# in eight runs at 1,024 keys where one run takes 8.8; in the step that gained 0.2 % at batch 1,
# the second kernel's place in the chain costing what its work-groups save: not taken.)
SPLIT_BYTES = 384 << 10
RUN_BYTES = 128 << 10
# A prompt step with few tiles of queries (a chunk of a prompt) cuts the keys of every tile into runs
# of at least this many blocks of 64 keys for every 256 tokens of the step (prompt_runs).
PROMPT_RUN_BLOCKS = 8
PROMPT_RUN_MIN_CONTEXT = 1024      # no runs in steps whose class of context is this or less: they gain from some 2,000 keys on


@register("mixer", "attention")
class CausalSelfAttention(Mixer):
    takes_deferred_norm = True
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        p = params
        self.width, self.heads, self.kv_heads = p["width"], p["heads"], p["kv_heads"]
        self.head_dim, self.scale, self.window = p["head_dim"], float(p["scale"]), int(p.get("window") or 0)
        if not p.get("causal", True):
            raise ValueError("attention: only causal attention runs from a cache")
        if self.head_dim <= 0:
            raise ValueError(f"attention: head size {self.head_dim} must be positive")
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"attention: {self.heads} query heads cannot share {self.kv_heads} key/value heads")
        self.n_q, self.n_kv = self.heads * self.head_dim, self.kv_heads * self.head_dim
        self.qkv_weight, self.qkv_bias = tensors["qkv_weight"], tensors.get("qkv_bias")
        self.out_weight, self.out_bias = tensors["out_weight"], tensors.get("out_bias")
        if tuple(self.qkv_weight.shape) != (self.n_q + 2 * self.n_kv, self.width):
            raise ValueError(f"attention: fused projection is {tuple(self.qkv_weight.shape)}, "
                             f"expected {(self.n_q + 2 * self.n_kv, self.width)}")
        if tuple(self.out_weight.shape) != (self.width, self.n_q):
            raise ValueError(f"attention: output projection is {tuple(self.out_weight.shape)}, "
                             f"expected {(self.width, self.n_q)}")

        # The MFMA kernels take head sizes in steps of 16 (bfloat16: up to 128).  In float32 every other
        # size (any divisor of the width is a valid configuration, src/models/gpt2.rs:279-281) runs on
        # the plain product and the plain attention kernel, which take any head size up to 256;
        # bfloat16 has no such kernels and says so here, before anything is built.
        bf16 = self.qkv_weight.dtype == torch.bfloat16
        if bf16 and (self.head_dim % 16 != 0 or self.head_dim > 128):
            raise ValueError(f"attention: the bfloat16 kernels take head sizes 16, 32, ... 128, not {self.head_dim}; "
                             f"load the model with dtype float32, which takes any head size up to 256")
        if self.head_dim > 256:
            raise ValueError(f"attention: head size {self.head_dim} is beyond 256, the most any kernel here takes")
        self.plain_only = self.head_dim % 16 != 0
        if self.plain_only:
            self.takes_deferred_norm = False       # the plain product reads row-major, normalised rows

        # second copies for decode steps, which read the weights and little else
        self.qkv_packed = K.PackedWeight(self.qkv_weight) if self.qkv_weight.is_cuda else None
        self.out_packed = packed_for_stream(self.out_weight) if self.out_weight.is_cuda else None

    def kv_spec(self):
        return KVSpec(self.kv_heads, self.head_dim, self.window)

    def kernel_modules(self, dtype):
        if self.plain_only:
            return ()
        if dtype == torch.bfloat16:
            return (f"attention_bf16_hd{self.head_dim}",)
        return ("attention_f32",) if self.head_dim <= 128 else ()

    def decode_runs(self, step, device):
        """Into how many runs a decode step's keys are cut: planned for the step's class of
        context, not its exact lengths, so that every step of a class runs the same kernels."""
        if not step.decode:
            return 1
        keys = min(step.context_limit, self.window + 32) if self.window else step.context_limit
        pair_bytes = keys * self.head_dim * 2 * (2 if step.dtype_is_bf16 else 4)     # one head's keys and values
        if pair_bytes <= SPLIT_BYTES:
            return 1
        pairs = step.n_seqs * self.kv_heads
        return max(1, min(compute_units(device) // pairs, pair_bytes // RUN_BYTES, 64))

    def prompt_runs(self, step, device):
        """Into how many runs a prompt step's query tiles cut their keys: a chunk of a prompt behind
        a long context has few tiles of 128 queries (a work-group each) and many keys for each, so
        the keys are shared out until the work-groups fill the chip, a run keeping at least
        ``PROMPT_RUN_BLOCKS`` blocks of keys.  Planned from what the steps that share a launch list
        have in common (most tokens, sequences, the class of context), like ``decode_runs``.
        Measured at 25 heads of 64, a chunk of 256 tokens, us a call with 1 / 2 / 4 / 5 runs: behind
        1,024 tokens 16.6 / 16.9 / 17.3 / 18.0, 2,048: 25.9 / 21.9 / 20.4 / 20.8, 4,096: 45.7 / 31.9 /
        25.5 / 25.3, 8,192: 84.5 / 51.9 / 35.6 / 33.7; two sequences (100 work-groups) 4,096: 48.1 /
        36.9, 8,192: 88.4 / 57.7."""
        if step.decode or not step.dtype_is_bf16 or self.head_dim != 64 or self.window or self.plain_only:
            return 1
        if step.context_limit <= PROMPT_RUN_MIN_CONTEXT:
            return 1
        tiles = -(-step.token_capacity // 128) + step.n_seqs - 1          # at most so many hold queries
        blocks = PROMPT_RUN_BLOCKS * -(-step.token_capacity // 256)       # (joining costs by the token)
        return max(1, min(compute_units(device) // (tiles * self.heads), step.context_limit // (64 * blocks), 8))

    def forward(self, h, step, memory, stream):
        tokens = h.shape[0]
        kv = memory.kv()
        if memory.writes and step.dtype_is_bf16 and not self.plain_only and \
                K.prompt_products_in_library(tokens, self.n_q + 2 * self.n_kv, self.width,
                                             h.stride(0) if hasattr(h, "stride") else self.width, scatters=True):
            # a prompt: the vendor's library makes the whole projection, then keys and values are
            # copied into the cache; the queries are read where they lie
            qkv = step.buffer("attention.qkv", tokens, self.n_q + 2 * self.n_kv, step.dtype)
            K.gemm(h, self.qkv_weight, K.epilogue_store(qkv, self.qkv_bias))
            K.kv_copy(qkv[:, self.n_q:self.n_q + self.n_kv], qkv[:, self.n_q + self.n_kv:], step.tok_seq,
                      step.tok_pos, kv, to_cache=True)
            q = qkv[:, :self.n_q]
        elif memory.writes:
            q = step.buffer("attention.q", tokens, self.n_q, step.dtype)
            K.gemm(h, self.qkv_weight,
                   K.epilogue_qkv(q, self.n_q, self.n_kv, kv, step.tok_seq, step.tok_pos, self.qkv_bias),
                   packed=self.qkv_packed, impl="plain" if self.plain_only else "auto")
        else:   # the keys and values of another layer are read; only the queries are projected
            q = step.buffer("attention.q", tokens, self.n_q, step.dtype)
            bias = self.qkv_bias[:self.n_q] if self.qkv_bias is not None else None
            K.gemm(h, self.qkv_weight[:self.n_q], K.epilogue_store(q, bias))
        if step.decode and step.dtype_is_bf16 and K.Chunked.wanted(tokens) \
                and self.head_dim <= 128 and self.heads // self.kv_heads <= 16:
            mixed = K.Chunked.take(step, "attention.mixed", tokens, self.n_q, step.dtype)    # the layout the next product reads fastest
        else:
            mixed = step.buffer("attention.mixed", tokens, self.n_q, step.dtype)
        partial, runs, prompt_runs = None, self.decode_runs(step, h.device), self.prompt_runs(step, h.device)
        if runs > 1:
            partial = step.buffer("attention.partial", step.n_seqs * self.heads * runs, self.head_dim + 2, "float32")
        elif prompt_runs > 1:
            partial = step.buffer("attention.partial", tokens * self.heads * prompt_runs, self.head_dim + 2, "float32")
        args = K.attention_args(q, mixed, kv, step.tok_seq, step.tok_pos, step.seq_off, step.seq_start,
                                self.heads, step.n_seqs, step.max_count, self.scale, self.window, partial,
                                runs=prompt_runs if prompt_runs > 1 else None)
        K.attention(args, step.dtype, step.decode, impl="plain" if self.plain_only else "auto")
        stream.add_product(step, mixed, self.out_weight, self.out_bias, packed=self.out_packed)
