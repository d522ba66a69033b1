"""Helpers of the GPU kernel tests: a paged cache filled from plain rows, and plain references."""

import math

import torch

from burn_transformers_amd.kernels import library as K

BLOCK = 64


class PagedCase:
    """Sequences with lengths ``totals`` whose last ``counts`` tokens are this step's; keys and
    values are random rows [tokens_total, kv_heads * head_dim] written into shuffled blocks."""

    def __init__(self, totals, counts, kv_heads, head_dim, dtype, device, seed=0, poison=False):
        gen = torch.Generator().manual_seed(seed)
        self.totals, self.counts = list(totals), list(counts)
        self.kv_heads, self.head_dim, self.dtype, self.device = kv_heads, head_dim, dtype, device
        n_seqs = len(totals)
        self.max_blocks = max((t + BLOCK - 1) // BLOCK for t in totals) + 1
        need = sum((t + BLOCK - 1) // BLOCK for t in totals)
        n_blocks = need + 3
        order = torch.randperm(n_blocks, generator=gen).tolist()
        table = torch.zeros(n_seqs, self.max_blocks, dtype=torch.int32)
        self.block_lists = []
        for s, t in enumerate(totals):
            blocks = [order.pop() for _ in range((t + BLOCK - 1) // BLOCK)]
            table[s, :len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
            self.block_lists.append(blocks)
        shape = (n_blocks, kv_heads, BLOCK, head_dim)
        fill = float("nan") if poison else 0.0
        self.keys = torch.full(shape, fill, dtype=dtype, device=device)
        self.values = torch.full(shape, fill, dtype=dtype, device=device)
        self.table = table.to(device)
        width = kv_heads * head_dim
        self.k_rows = [(torch.randn(t, width, generator=gen) * 0.7).to(dtype) for t in totals]
        self.v_rows = [(torch.randn(t, width, generator=gen)).to(dtype) for t in totals]
        # all positions through the kv_copy kernel
        seq = torch.cat([torch.full((t,), s, dtype=torch.int32) for s, t in enumerate(totals)]).to(device)
        pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in totals]).to(device)
        K.kv_copy(torch.cat(self.k_rows).to(device), torch.cat(self.v_rows).to(device), seq, pos, self.view(), True)
        # this step's tokens
        self.starts = [t - c for t, c in zip(totals, counts)]
        self.tok_seq = torch.cat([torch.full((c,), s, dtype=torch.int32) for s, c in enumerate(counts)]).to(device)
        self.tok_pos = torch.cat([torch.arange(st, st + c, dtype=torch.int32)
                                  for st, c in zip(self.starts, counts)]).to(device)
        offsets = [0]
        for c in counts:
            offsets.append(offsets[-1] + c)
        self.seq_off = torch.tensor(offsets, dtype=torch.int32, device=device)
        self.seq_start = torch.tensor(self.starts, dtype=torch.int32, device=device)
        self.n_tokens = offsets[-1]

    def view(self):
        return K.KvView(keys=self.keys.data_ptr(), values=self.values.data_ptr(), blocks=self.table.data_ptr(),
                        max_blocks=self.max_blocks, kv_heads=self.kv_heads, head_dim=self.head_dim,
                        block_stride=self.kv_heads * BLOCK * self.head_dim, head_stride=BLOCK * self.head_dim)

    def read_back(self):
        """Keys and values of every position, through the kv_copy kernel."""
        seq = torch.cat([torch.full((t,), s, dtype=torch.int32) for s, t in enumerate(self.totals)]).to(self.device)
        pos = torch.cat([torch.arange(t, dtype=torch.int32) for t in self.totals]).to(self.device)
        width = self.kv_heads * self.head_dim
        k = torch.empty(sum(self.totals), width, dtype=self.dtype, device=self.device)
        v = torch.empty_like(k)
        K.kv_copy(k, v, seq, pos, self.view(), False)
        return k, v

    def reference(self, q, q_heads, scale, window=0):
        """float64 attention of the step's queries q [tokens, q_heads * head_dim] (CPU)."""
        hd, group = self.head_dim, q_heads // self.kv_heads
        out = torch.zeros(self.n_tokens, q_heads * hd, dtype=torch.float64)
        q = q.detach().cpu().to(torch.float64)
        row = 0
        for s, (total, count) in enumerate(zip(self.totals, self.counts)):
            k = self.k_rows[s].to(torch.float64).view(total, self.kv_heads, hd)
            v = self.v_rows[s].to(torch.float64).view(total, self.kv_heads, hd)
            for i in range(count):
                pos = total - count + i
                lo = max(0, pos - window + 1) if window else 0
                for h in range(q_heads):
                    qv = q[row, h * hd:(h + 1) * hd]
                    scores = (k[lo:pos + 1, h // group] @ qv) * scale
                    w = torch.softmax(scores, dim=0)
                    out[row, h * hd:(h + 1) * hd] = w @ v[lo:pos + 1, h // group]
                row += 1
        return out


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def gelu_erf(x):
    return x * (1.0 + torch.erf(x / math.sqrt(2.0))) / 2.0
