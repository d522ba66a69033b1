"""Token selection on the GPU: greedy (lowest index of the maximum) or temperature sampling by
inverse CDF with SplitMix64 uniforms, and the log-probability of the chosen token under the
distribution that was used (src/generation.rs:655-664, 732-743, 1148-1165).  A configuration
that asks for more (logit bias, repetition / presence / frequency penalties, banned n-grams,
end-of-sequence held back until min_new_tokens, top-k, top-p, min-p; src/generation.rs:18-44)
goes through one kernel that holds a row in registers and applies them in the reference's order.

Draw numbering follows the reference (src/generation.rs:667-699): every selection over a batch
that started with B rows reserves B draws, finished rows included, so the row that started as
number b uses draw  s * B + b  in step s.
"""

import torch

from ..kernels import library as K

_MASK64 = 2 ** 64 - 1


def splitmix64(seed, index):
    """Output ``index`` of the stream (src/generation/random.rs:232-237); host twin of the kernel."""
    value = (seed + 0x9E3779B97F4A7C15 * ((index + 1) & _MASK64)) & _MASK64
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK64
    return value ^ (value >> 31)


def interior_unit(bits):
    """The uniform in (0, 1) the kernel derives from 64 mixed bits (random.rs:244-247)."""
    return ((bits >> 41) + 0.5) / float(1 << 23)


class Sampler:
    def __init__(self, config, batch_rows, device, vocabulary_size=None, prompts=None):
        """``prompts`` (token ids of every row of the batch) are needed when the configuration asks
        for anything that depends on what a row has held so far (penalties, n-gram bans)."""
        self.config, self.batch_rows, self.device = config, batch_rows, device
        self.selections = 0
        # ids and log-probabilities share one buffer so that they come back in one copy
        self.packed = torch.zeros((2, batch_rows), dtype=torch.int32, device=device)
        self.ids, self.logp = self.packed[0], self.packed[1].view(torch.float32)
        self.host = torch.zeros((2, batch_rows), dtype=torch.int32).pin_memory()
        self._arrived = torch.cuda.Event()     # the copy of the latest selection into `host`
        self._launched = 0                     # rows of the selection that `result` has not fetched yet
        self.history = self.bias = None
        if vocabulary_size is not None and config.processes_logits(vocabulary_size):
            from .history import TokenHistory
            self.history = TokenHistory(config, vocabulary_size, prompts if prompts is not None
                                        else [[] for _ in range(batch_rows)], device)
            if config.logit_bias:
                bias = torch.zeros(vocabulary_size, dtype=torch.float32)
                for token, value in config.logit_bias.items():
                    bias[token] = value
                self.bias = bias.to(device)

    @property
    def pipelined(self):
        """True where a selection needs nothing from the host but the rows' numbers: it can then be
        started (``launch``) and fetched later (``result``), and the chosen ids can feed the next
        step from the GPU (``device_ids``) before the host has seen them."""
        return self.history is None

    def launch(self, logits, rows):
        """Starts the selection of one token per row and its copy to the host; returns at once."""
        if self.history is not None:
            raise RuntimeError("a selection that depends on what the rows have held so far cannot run ahead of the host")
        count = len(rows)
        config = self.config
        draw_rows = None
        if config.sampling:
            draw_rows = torch.tensor(rows, dtype=torch.int32).to(self.device, non_blocking=True)
        K.sample(logits, self.ids[:count], self.logp[:count],
                 temperature=float(config.temperature) if config.sampling else None,
                 seed=config.seed, first_draw=self.selections * self.batch_rows, draw_rows=draw_rows)
        self.selections += 1
        self.host.copy_(self.packed, non_blocking=True)
        self._arrived.record()
        self._launched = count

    def device_ids(self, count):
        """The ids of the latest selection where they were chosen: int32 [count] on the GPU."""
        return self.ids[:count]

    def result(self):
        """(ids, log-probabilities) of the selection ``launch`` started, as Python lists; waits for
        their copy.  This is the step's one readback."""
        count, self._launched = self._launched, 0
        self._arrived.synchronize()
        return self.host[0, :count].tolist(), self.host[1].view(torch.float32)[:count].tolist()

    def select(self, logits, rows):
        """One token for each row of ``logits`` (float32 [len(rows), vocab]); ``rows`` are the rows'
        numbers in the batch as it started.  Returns (ids, log-probabilities) as Python lists."""
        count = len(rows)
        config = self.config
        first_draw = self.selections * self.batch_rows
        if self.history is None:
            self.launch(logits, rows)
            return self.result()
        else:
            # one small upload: the rows' numbers, then where each row's banned tokens start, then those
            banned = [self.history.banned(row) for row in rows]
            offsets = [0]
            for tokens in banned:
                offsets.append(offsets[-1] + len(tokens))
            flat = list(rows) + offsets + [t for tokens in banned for t in tokens]
            table = torch.tensor(flat, dtype=torch.int32).to(self.device, non_blocking=True)
            has_bans = offsets[-1] > 0
            K.select_processed(
                logits, self.ids[:count], self.logp[:count], bias=self.bias,
                counts_all=self.history.counts_all if config.repetition_penalty != 1.0 else None,
                counts_add=self.history.additive_counts, batch_rows=table[:count],
                ban_ids=table[2 * count + 1:] if has_bans else None,
                ban_offsets=table[count:2 * count + 1] if has_bans else None,
                repetition=float(config.repetition_penalty), presence=float(config.presence_penalty),
                frequency=float(config.frequency_penalty),
                temperature=float(config.temperature) if config.sampling else None,
                clamp=config.adjusts_logits or (config.sampling and config.temperature < 1.0),
                top_k=config.top_k if config.sampling and config.top_k is not None else 0,
                top_p=float(config.top_p) if config.sampling and config.top_p is not None else 1.0,
                min_p=float(config.min_p) if config.sampling and config.min_p is not None else 0.0,
                seed=config.seed, first_draw=first_draw)
        self.selections += 1
        self.host.copy_(self.packed)                  # synchronous: the kernels above have finished after it
        ids = self.host[0, :count].tolist()
        if self.history is not None:
            self.history.record(list(rows), ids)
        return ids, self.host[1].view(torch.float32)[:count].tolist()
